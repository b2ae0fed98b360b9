// Whole-solve kernel for right-hand sides on a periodic N x N grid (reaction-diffusion,
// F = N*N state values per sample; N = 16, 32 or 64 in float32 or float64, 128 in float32): one workgroup per sample,
// of N*N/4 threads up to N = 64 and of 1024 threads on the 128 x 128 grid.
//
// Thread t owns the four consecutive cells 4t..4t+3 of the row-major grid (on the 128 x 128 grid: of each of its four
// bands of 32 rows, so that every wavefront still holds one chunk of 256 consecutive cells per band) and keeps
// their state (y, the seven stage derivatives, the dense-output coefficients) in
// registers for the whole solve.  Only the stage input travels through LDS, double
// buffered, so that the five-point stencil can read its neighbours: one barrier per
// right-hand side evaluation.  Norms over the row are block reductions in a fixed
// order (the order of wave_row_norm in tode_solve.h: per-thread chain over its four
// values, butterfly over the wavefront, wavefront sums added in order), so that this
// kernel and the per-call operators produce the same bits.  Every thread of the
// workgroup carries the same scalar state (t, dt, error ratio, counters), computed
// redundantly from the same reduced values: there is no divergence inside a sample.
//
// The dense output is what this kernel is bound by: every evaluation point is one
// coalesced 4*F-byte row of ys, written with 16-byte stores straight from registers.
//
// Same contract as the fast kernels: the common case only; anything else (a
// non-success status, max_steps reached, evaluation times that are not monotone in
// the direction of time, a sample that does not land on t_end) raises
// TODE_FLAG_NEEDS_GENERAL and leaves the outputs unspecified.
#include <limits.h>

#include "tode_solve.h"

namespace tode {

struct GridOut {
    int64_t *n_steps, *n_accepted, *n_initialized, *status;
};

template <typename T, int NW, int R> struct GridShared {
    T xch[2][R * NW * 256];  // stage input, double buffered
    T red[2][R][NW][2];      // chunk sums of up to two reductions, double buffered
    T xs[NW * 64];           // positions within the step of the evaluation points it passed (one per thread and round)
    int passed[NW];          // per wavefront: how many of its threads' candidate points the step passed
    T handed;                // a scalar of the sample that one wavefront worked out for all (by_one_wavefront)
};

// Four consecutive values, moved with the widest loads and stores their alignment allows.
template <typename T> struct alignas(4 * sizeof(T)) Four {
    T x, y, z, w;
};
template <typename T> __device__ __forceinline__ void load4(const T *from, T (&v)[4]) {
    const Four<T> f = *reinterpret_cast<const Four<T> *>(from);
    v[0] = f.x, v[1] = f.y, v[2] = f.z, v[3] = f.w;
}
template <typename T> __device__ __forceinline__ void store4(T *to, const T (&v)[4]) { *reinterpret_cast<Four<T> *>(to) = Four<T>{v[0], v[1], v[2], v[3]}; }

// Sum over the row of two per-thread partial sums per band, in the fixed order: the chunk of 256 cells that wavefront w
// holds of band r is chunk r * NW + w of the row, and the chunk sums are added in that order.
template <typename T, int NW, int R> __device__ __forceinline__ void block_sum2(GridShared<T, NW, R> &sh, int &slot, const T (&a)[R], const T (&b)[R], T &A, T &B) {
    const int wave = threadIdx.x >> 6;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        T u = a[r], v = b[r];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            u = u + __shfl_xor(u, off);
            v = v + __shfl_xor(v, off);
        }
        if ((threadIdx.x & 63) == 0) {
            sh.red[slot][r][wave][0] = u;
            sh.red[slot][r][wave][1] = v;
        }
    }
    lds_barrier();
    A = 0;
    B = 0;
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            A = A + sh.red[slot][r][w][0];
            B = B + sh.red[slot][r][w][1];
        }
    slot ^= 1;
}

// A scalar of the sample that takes hundreds of instructions (a power): worked out by the first wavefront alone and
// handed round in LDS, where otherwise all NW wavefronts would work it out, four to a SIMD one after the other.  Same
// arithmetic on the same operands: same bits.  (Between two uses lies at least one other barrier of the workgroup, so
// nobody still reads the word when it is written again.)
template <typename T, typename Compute> __device__ __forceinline__ T by_one_wavefront(T &word, Compute compute) {
    if (threadIdx.x < 64) {
        const T value = compute();
        if (threadIdx.x == 0) word = value;
    }
    lds_barrier();
    return word;
}

// du/dt = D * lap(u) + u * (1 - u) on the periodic grid; each operation rounds on its own, in the
// order of the torch expression  (((up + down) + left) + right) - 4u,  D * lap + u * (1 - u).
template <typename T, int N, int NW, int R>
__device__ __forceinline__ void grid_rhs(GridShared<T, NW, R> &sh, int &buf, T D, const T (&u)[R][4], T (&out)[R][4]) {
    const int t = threadIdx.x;
    constexpr int PER_ROW = N / 4, BAND = N * N / R, BAND_ROWS = N / R;
    const int rl = t / PER_ROW, c0 = 4 * (t - rl * PER_ROW);
    T *x = sh.xch[buf];
#pragma unroll
    for (int r = 0; r < R; ++r) store4<T>(x + r * BAND + 4 * t, u[r]);
    lds_barrier();
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int row = r * BAND_ROWS + rl;
        const int ru = (row + N - 1) & (N - 1), rd = (row + 1) & (N - 1);
        T ups[4], dns[4];
        load4<T>(x + ru * N + c0, ups);
        load4<T>(x + rd * N + c0, dns);
        const T lf = x[row * N + ((c0 + N - 1) & (N - 1))];
        const T rt = x[row * N + ((c0 + 4) & (N - 1))];
        const T lfs[4] = {lf, u[r][0], u[r][1], u[r][2]}, rts[4] = {u[r][1], u[r][2], u[r][3], rt};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const T lap = (((ups[j] + dns[j]) + lfs[j]) + rts[j]) - ((T)4 * u[r][j]);
            const T diff = D * lap;
            const T react = u[r][j] * ((T)1 - u[r][j]);
            out[r][j] = diff + react;
        }
    }
    buf ^= 1;
}

constexpr int grid_bands(int n) { return n * n / 4 > 1024 ? n * n / 4 / 1024 : 1; }

// END_ONLY: no evaluation points (a compile-time constant, so that the usual kernel carries none of that mode's code).
template <typename T, int METHOD, int CTRL, int N, bool END_ONLY>
__global__ void __launch_bounds__(N *N / 4 / grid_bands(N)) solve_grid_kernel(const SolveParams<T> p, const GridOut o) {
    using Tab = typename std::conditional<METHOD == 1, Tsit5Tab, Dopri5Tab>::type;
    constexpr int F = N * N, R = grid_bands(N), NT = F / 4 / R, NW = NT / 64, BAND = F / R;
    __shared__ GridShared<T, NW, R> sh;
    extern __shared__ __align__(16) unsigned char dyn[];
    T *te_s = reinterpret_cast<T *>(dyn);  // [E] evaluation times of this sample

    const int tid = threadIdx.x;
    const long long b = blockIdx.x;
    // Without evaluation points (the end point alone, adjoints.py:296-311) t_end is the sample's one point: ys takes the
    // dense output of its last step there and y_idle its final state; the caller picks per sample (tode_select_end_point).
    constexpr bool end_only = END_ONLY;
    const int E = end_only ? 1 : p.n_eval;
    const CtrlParams<T> &cp = p.cp;
    const T sf = (T)__builtin_sqrt((double)F);
    int buf = 0, slot = 0;

    for (int e = tid; e < E; e += NT) te_s[e] = end_only ? p.t_end[b * p.te_stride] : p.t_eval[b * E + e];
    const T ts = p.t_start[b * p.ts_stride], te = p.t_end[b * p.te_stride];
    const T dir = (te > ts) ? (T)1 : (T)-1;
    const T tlo = tmin(ts, te), thi = tmax(te, ts);
    const T D = p.params[b];
    T y[R][4], k[7][R][4];
#pragma unroll
    for (int r = 0; r < R; ++r) load4<T>(p.y0 + b * F + r * BAND + 4 * tid, y[r]);
    __syncthreads();  // te_s

    // evaluation times that are not monotone in the sample's direction: each thread looks at its share of the neighbours
    int disorder = 0;
    for (int e = 1 + tid; e < E; e += NT) disorder |= !(dir * te_s[e] >= dir * te_s[e - 1]);
    bool bail = __syncthreads_or(disorder) != 0;

    // ---- first step size (step_size_controllers.py:431-490, 776-835) ----
    T t = ts, dt;
    grid_rhs<T, N, NW, R>(sh, buf, D, y, k[0]);
    if (p.dt0) {
        dt = p.dt0[b];
    } else {
        T inv[R][4], a0[R], a1[R], A0, A1;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            a0[r] = 0, a1[r] = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                inv[r][j] = inv_scale(cp.atol, cp.rtol, y[r][j]);
                const T x0 = (y[r][j] * inv[r][j]) / sf, x1 = (k[0][r][j] * inv[r][j]) / sf;
                a0[r] = fma_(x0, x0, a0[r]);
                a1[r] = fma_(x1, x1, a1[r]);
            }
        }
        block_sum2<T, NW, R>(sh, slot, a0, a1, A0, A1);
        const T d0 = sqrt_(A0), d1 = sqrt_(A1);
        T h0 = (d0 < (T)1e-5 || d1 < (T)1e-5) ? (T)1e-6 : ((T)0.01 * d0) / d1;
        h0 = tmin(h0, abs_(te - ts));
        T y1[R][4], f1[R][4];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < 4; ++j) y1[r][j] = fma_(dir * h0, k[0][r][j], y[r][j]);
        grid_rhs<T, N, NW, R>(sh, buf, D, y1, f1);
        T a2[R], none[R], A2, unused;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            a2[r] = 0, none[r] = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const T df = f1[r][j] - k[0][r][j];
                const T x2 = (df * inv[r][j]) / sf;
                a2[r] = fma_(x2, x2, a2[r]);
            }
        }
        block_sum2<T, NW, R>(sh, slot, a2, none, A2, unused);
        dt = by_one_wavefront(sh.handed, [&] { return initial_finish<T>(CTRL == 1 ? TODE_CTRL_PID : TODE_CTRL_INTEGRAL, 1.0 / 5.0, dir, h0, d1, sqrt_(A2)); });
    }
    dt = tclamp(dt, tlo - t, thi - t);

    int cursor = 0, n_steps = 0, n_acc = 0;
    if (E > 0 && te_s[0] == ts) {
#pragma unroll
        for (int r = 0; r < R; ++r) store4<T>(p.ys + (b * E) * F + r * BAND + 4 * tid, y[r]);
        cursor = 1;
    }
    T prev = 1, pprev = 1;

    // A sample that has landed past t_end (t + (t_end - t) rounded upwards) keeps stepping in the reference's later
    // iterations with the clamped step t_end - t, which is seen only in the status of that step: the workgroup
    // computes that step once more and looks at its status.
    bool idle = false, idle_done = false;
    while (!bail) {
        // ---- stages (runge_kutta.py:255-263) ----
        const T t0 = t;
        T y1[R][4];
#pragma unroll
        for (int i = 1; i < 7; ++i) {
            T yi[R][4];
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    T s = 0;
#pragma unroll
                    for (int jj = 0; jj < i; ++jj) s = fma_((T)Tab::a[i][jj], k[jj][r][j], s);
                    yi[r][j] = fma_(dt, s, y[r][j]);
                }
            grid_rhs<T, N, NW, R>(sh, buf, D, yi, k[i]);
            if (i == 6) {
#pragma unroll
                for (int r = 0; r < R; ++r)
#pragma unroll
                    for (int j = 0; j < 4; ++j) y1[r][j] = yi[r][j];
            }
        }

        // ---- error ratio (runge_kutta.py:267, step_size_controllers.py:389-395); long rows: fused sums ----
        T part[R], none[R], total, unused;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            part[r] = 0, none[r] = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                T err = 0;
#pragma unroll
                for (int s = 0; s < 7; ++s) err = fma_(dt * (T)Tab::b_err[s], k[s][r][j], err);
                const T m = tmax(abs_(y[r][j]), abs_(y1[r][j]));
                const T x = (abs_(err) / fma_(cp.rtol, m, cp.atol)) / sf;
                part[r] = fma_(x, x, part[r]);
            }
        }
        block_sum2<T, NW, R>(sh, slot, part, none, total, unused);
        const T ratio = tmax(sqrt_(total), (T)1e-38);
        const bool accept = ratio < (T)1;
        T dt_next = dt * by_one_wavefront(sh.handed, [&] { return dt_factor<T, CTRL>(cp, ratio, prev, pprev); });
        const int status = limit_dt<T>(cp, ratio, dt_next);
        if (idle) {
            bail = status != 0;
            if (end_only && !bail) {  // the end point of such a sample is this step's interpolant at t_end
                const T x = unit_time(te, t0, t0 + dt);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    T out[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        T ks[7], q[5][1];
#pragma unroll
                        for (int s = 0; s < 7; ++s) ks[s] = k[s][r][j];
                        quartic_elem<T, METHOD>(dt, y[r][j], y1[r][j], ks, true, q);
                        T v = q[4][0];
#pragma unroll
                        for (int pw = 3; pw >= 0; --pw) v = fma_(v, x, q[pw][0]);
                        out[j] = v;
                    }
                    store4<T>(p.y_idle + b * F + r * BAND + 4 * tid, out);
                }
                idle_done = true;
            }
            break;
        }

        const T t_new = accept ? (t0 + dt) : t0;
        const bool running_new = fma_(dir, t_new, -dir * te) < (T)0;
        n_steps += 1;
        n_acc += accept ? 1 : 0;

        // ---- dense output at the evaluation points this step passed (adjoints.py:215-234) ----
        // Which points those are and where each lies within the step, x = (t_eval - t0) / (t1 - t0), is the same for
        // every cell of the sample: worked out once per point (thread i looks at point cursor + i; the evaluation times
        // are monotone, so the passed ones are the first `count` of them) and handed round in LDS, instead of a division
        // and a comparison per thread and point.  What every thread then does per point is the polynomial of its four
        // cells and one 16-byte store.  (Band by band: the coefficients of one band at a time are alive.)
        if (cursor < E && fma_(dir, t_new, -dir * te_s[cursor]) >= (T)0) {
            const T t1 = t0 + dt;
            while (true) {
                const int mine = cursor + tid;
                const bool ok = mine < E && fma_(dir, t_new, -dir * te_s[mine]) >= (T)0;
                if (ok) sh.xs[tid] = unit_time(te_s[mine], t0, t1);
                const unsigned long long votes = __ballot(ok);
                if ((tid & 63) == 0) sh.passed[tid >> 6] = __popcll(votes);
                lds_barrier();
                int count = 0;
#pragma unroll
                for (int w = 0; w < NW; ++w) count += sh.passed[w];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    T q[4][5][1];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        T ks[7];
#pragma unroll
                        for (int s = 0; s < 7; ++s) ks[s] = k[s][r][j];
                        quartic_elem<T, METHOD>(dt, y[r][j], y1[r][j], ks, true, q[j]);
                    }
                    T *row = p.ys + (b * E + cursor) * F + r * BAND + 4 * tid;
#pragma unroll 4
                    for (int i = 0; i < count; ++i) {
                        const T x = sh.xs[i];
                        T out[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            T v = q[j][4][0];
#pragma unroll
                            for (int pw = 3; pw >= 0; --pw) v = fma_(v, x, q[j][pw][0]);
                            out[j] = v;
                        }
                        store4<T>(row + (long long)i * F, out);
                    }
                }
                cursor += count;
                if (count < NT || cursor >= E) break;
                lds_barrier();  // (a step that passed more points than the workgroup has threads: another round)
            }
        }

        // ---- state update (adjoints.py:150-155, 247-255) ----
        if (accept) {
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    y[r][j] = y1[r][j];
                    k[0][r][j] = k[6][r][j];
                }
        }
        t = t_new;
        dt = tclamp(running_new ? dt_next : dt, tlo - t, thi - t);
        if (CTRL == 1 && running_new && accept) {
            pprev = prev;
            prev = ratio;
        }
        if (status != 0 || n_steps >= p.max_steps || n_steps >= TODE_HARD_STEP_LIMIT) {
            bail = true;
            break;
        }
        if (!running_new) {
            // a sample that ends on a non-finite value shows up in later iterations of the reference loop: not the
            // common case; one that landed past t_end is looked at in one more iteration
            int odd = 0;
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int j = 0; j < 4; ++j) odd |= !settles_(y[r][j], k[0][r][j]);
            if (__syncthreads_or(odd)) bail = true;
            if (bail || t == te) break;
            idle = true;
        }
    }

    if (end_only && !idle_done) {
#pragma unroll
        for (int r = 0; r < R; ++r) store4<T>(p.y_idle + b * F + r * BAND + 4 * tid, y[r]);  // the final state
    }
    if (tid == 0) {
        o.n_steps[b] = n_steps;
        o.n_accepted[b] = n_acc;
        o.n_initialized[b] = cursor;
        o.status[b] = 0;
        if (n_steps > 0) atomicMax(&p.flags[TODE_FLAG_MAX_ITERATIONS], n_steps);
        if (bail) atomicMax(&p.flags[TODE_FLAG_NEEDS_GENERAL], 1);
    }
    publish_flags(p);
}

template <typename T, int METHOD, int CTRL, int N> static int launch_grid(const tode_solve_args &a, const tode_controller &c, const GridOut &o, hipStream_t stream) {
    SolveParams<T> p = make_params<T>(a, c);
    reset_flags(a.flags, stream);
    if (a.batch == 0) return check_hip(hipGetLastError(), "tode_solve_builtin_fast launch");
    const size_t lds = (size_t)(a.n_eval > 0 ? a.n_eval : 1) * sizeof(T);
    timing_before(stream, "tode::solve_grid_kernel");
    if (a.n_eval > 0)
        hipLaunchKernelGGL((solve_grid_kernel<T, METHOD, CTRL, N, false>), dim3((unsigned)a.batch), dim3(N * N / 4 / grid_bands(N)), lds, stream, p, o);
    else
        hipLaunchKernelGGL((solve_grid_kernel<T, METHOD, CTRL, N, true>), dim3((unsigned)a.batch), dim3(N * N / 4 / grid_bands(N)), lds, stream, p, o);
    timing_after(stream);
    return check_hip(hipGetLastError(), "tode_solve_builtin_fast launch");
}

template <typename T, int N> static int grid_mc(const tode_solve_args &a, const tode_controller &c, const GridOut &o, hipStream_t s) {
    if (a.method == TODE_DOPRI5 && c.kind == TODE_CTRL_INTEGRAL) return launch_grid<T, 0, 0, N>(a, c, o, s);
    if (a.method == TODE_DOPRI5 && c.kind == TODE_CTRL_PID) return launch_grid<T, 0, 1, N>(a, c, o, s);
    if (a.method == TODE_TSIT5 && c.kind == TODE_CTRL_INTEGRAL) return launch_grid<T, 1, 0, N>(a, c, o, s);
    if (a.method == TODE_TSIT5 && c.kind == TODE_CTRL_PID) return launch_grid<T, 1, 1, N>(a, c, o, s);
    return fail(TODE_E_INVALID, "unknown method %d or controller kind %d", a.method, c.kind);
}

template <typename T> static int solve_grid(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s) {
    if (a.n_params != 1) return fail(TODE_E_INVALID, "reaction-diffusion needs one parameter (the diffusivity) per sample");
    if (a.n_eval > 8192) return fail(TODE_E_UNSUPPORTED, "n_eval=%d is too large for the grid kernel", a.n_eval);
    if (a.batch > INT_MAX) return fail(TODE_E_UNSUPPORTED, "batch too large");
    GridOut o{ns, na, ni, st};
    if (a.n_features == 64 * 64) return grid_mc<T, 64>(a, c, o, s);
    if (a.n_features == 32 * 32) return grid_mc<T, 32>(a, c, o, s);
    if (a.n_features == 16 * 16) return grid_mc<T, 16>(a, c, o, s);  // (one wavefront per sample)
    if (sizeof(T) == 4 && a.n_features == 128 * 128) {
        // (128 KB of LDS for the double-buffered stage input leave 30 KB for the sample's evaluation times)
        if (a.n_eval > 4096) return fail(TODE_E_UNSUPPORTED, "n_eval=%d is too large for the grid kernel on the 128 x 128 grid", a.n_eval);
        return grid_mc<float, 128>(a, c, o, s);
    }
    return fail(TODE_E_UNSUPPORTED, "the grid kernel is built for 16 x 16, 32 x 32 and 64 x 64 grids (float32 also 128 x 128), got F=%d", a.n_features);
}

int solve_grid_f32(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s) {
    return solve_grid<float>(a, c, ns, na, ni, st, s);
}

int solve_grid_f64(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s) {
    return solve_grid<double>(a, c, ns, na, ni, st, s);
}

}  // namespace tode
