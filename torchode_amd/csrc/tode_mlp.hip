// Whole-solve kernel for a two-layer perceptron right-hand side shared by the batch,
//   f(t, y) = tanh([y, t] W1^T + b1) W2^T + b2,   y in R^64, 256 hidden units, float32,
// with both matrix products on the matrix cores (v_mfma_f32_16x16x4_f32).
//
// One workgroup of four wavefronts advances a tile of 16 samples.
//   * The weights never move after the prologue: every lane keeps, in registers, exactly
//     the B operands its wavefront feeds to the matrix cores -- wavefront w owns hidden
//     units 64w..64w+63 of the first layer (17 k-steps x 4 tiles = 68 registers) and output
//     features 16w..16w+15 of the second (64 k-steps = 64 registers).
//   * Layer 1: the stage input [16 x 65] goes to LDS once, every wavefront reads it as the
//     A operand and accumulates its four 16 x 16 tiles of hidden units; tanh; the hidden
//     tile [16 x 256] goes to LDS.  Layer 2: every wavefront reads the hidden tile as the A
//     operand and accumulates one 16 x 16 tile of outputs in four partial accumulators.
//     Two barriers per evaluation of f.
//   * The accumulator layout of the second layer is the layout of the solver state: lane
//     (q = lane/16, c = lane%16) of wavefront w holds feature 16w + c of samples 4q..4q+3,
//     for y, the seven stage derivatives and the dense-output coefficients.  Per-sample
//     scalars (t, dt, error ratio, counters) are carried redundantly by the 64 lanes that
//     share a sample.
//
// Same contract as the other fast kernels: the common case only; anything else raises
// TODE_FLAG_NEEDS_GENERAL and leaves the outputs unspecified.
#include <limits.h>

#include "tode_solve.h"

namespace tode {

typedef float mfma_acc __attribute__((ext_vector_type(4)));

struct MlpOut {
    int64_t *n_steps, *n_accepted, *n_initialized, *status;
};

constexpr int MLP_F = 64, MLP_H = 256, MLP_K1 = 68;  // 65 inputs padded to a multiple of 4
// LDS rows of the two A operands, stored so that what a lane feeds to the matrix cores is contiguous:
// lane (q, c) needs row c, columns 4 kk + q for all kk; column k sits at (k % 4) * (K / 4) + k / 4.
constexpr int MLP_XS = 4 * 17 + 4, MLP_HS = 4 * 64 + 4;  // row strides (floats), multiples of 4 for 16-byte reads
constexpr int MLP_TILE = 16;

struct __align__(16) MlpShared {
    float x[MLP_TILE * MLP_XS];
    float hid[MLP_TILE * MLP_HS];
    float red[2][4][MLP_TILE][2];  // per-wavefront partial sums of up to two per-sample reductions
};

struct MlpWeights {
    float w1[17][4];  // B operands of layer 1: W1[64w + 16 tile + c][4 kk + q]
    float b1[4];
    float w2[64];     // B operands of layer 2: W2[16w + c][4 kk + q]
    float b2;
};

// tanh(x) = 1 - 2 / (exp(2x) + 1) on the hardware exp2 and reciprocal: absolute error about 2e-7
// (the library tanhf costs several times the matrix products of a layer).  exp2 overflows to inf
// and underflows to 0 exactly where tanh saturates, so no range checks are needed.
__device__ __forceinline__ float mlp_tanh(float x) {
    const float e = __builtin_amdgcn_exp2f(x * 2.8853900817779268f);  // 2 / ln 2
    return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
}

// out[r] = f(tn[r], yi[r]) for the lane's four (sample, feature) pairs.
__device__ __forceinline__ void mlp_rhs(MlpShared &sh, const MlpWeights &W, const float (&tn)[4], const float (&yi)[4], float (&out)[4]) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, q = lane >> 4, c = lane & 15;
    {
        const int k = 16 * w + c;  // this lane's feature is input column k
#pragma unroll
        for (int r = 0; r < 4; ++r) sh.x[(4 * q + r) * MLP_XS + (k & 3) * 17 + (k >> 2)] = yi[r];
        if (w == 0 && c == 0) {
#pragma unroll
            for (int r = 0; r < 4; ++r) sh.x[(4 * q + r) * MLP_XS + (MLP_F & 3) * 17 + (MLP_F >> 2)] = tn[r];
        }
    }
    __syncthreads();
    // all A operands of the layer into registers first, so that the matrix cores never wait for LDS
    float a1[20];
    {
        const float *row = sh.x + c * MLP_XS + q * 17;  // 17 contiguous values (read as 20)
#pragma unroll
        for (int j = 0; j < 20; ++j) a1[j] = row[j];
    }
    asm volatile("" ::: "memory");
    mfma_acc acc1[4];
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) acc1[tile] = {W.b1[tile], W.b1[tile], W.b1[tile], W.b1[tile]};
#pragma unroll
    for (int kk = 0; kk < 17; ++kk) {
#pragma unroll
        for (int tile = 0; tile < 4; ++tile) acc1[tile] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1[kk], W.w1[kk][tile], acc1[tile], 0, 0, 0);
    }
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) {
        const int h = 64 * w + 16 * tile + c;
#pragma unroll
        for (int r = 0; r < 4; ++r) sh.hid[(4 * q + r) * MLP_HS + (h & 3) * 64 + (h >> 2)] = mlp_tanh(acc1[tile][r]);
    }
    __syncthreads();
    float a2[64];
    {
        const float4 *row = reinterpret_cast<const float4 *>(sh.hid + c * MLP_HS + q * 64);
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const float4 v = row[j];
            a2[4 * j] = v.x, a2[4 * j + 1] = v.y, a2[4 * j + 2] = v.z, a2[4 * j + 3] = v.w;
        }
    }
    asm volatile("" ::: "memory");
    mfma_acc acc2[4];
    acc2[0] = {W.b2, W.b2, W.b2, W.b2};
#pragma unroll
    for (int i = 1; i < 4; ++i) acc2[i] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int kk = 0; kk < 64; ++kk) acc2[kk & 3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a2[kk], W.w2[kk], acc2[kk & 3], 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 4; ++r) out[r] = (acc2[0][r] + acc2[1][r]) + (acc2[2][r] + acc2[3][r]);
}

// Per-sample sums over the 64 features of two quantities at once: 16 lanes of each wavefront by
// shuffles, the four wavefronts through LDS.  a, b: the lane's contributions for its 4 samples.
__device__ __forceinline__ void mlp_sum2(MlpShared &sh, int &slot, const float (&a)[4], const float (&b)[4], float (&A)[4], float (&B)[4]) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, q = lane >> 4, c = lane & 15;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        float u = a[r], v = b[r];
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) {
            u = u + __shfl_xor(u, off);
            v = v + __shfl_xor(v, off);
        }
        if (c == 0) {
            sh.red[slot][w][4 * q + r][0] = u;
            sh.red[slot][w][4 * q + r][1] = v;
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int s = 4 * q + r;
        A[r] = (sh.red[slot][0][s][0] + sh.red[slot][1][s][0]) + (sh.red[slot][2][s][0] + sh.red[slot][3][s][0]);
        B[r] = (sh.red[slot][0][s][1] + sh.red[slot][1][s][1]) + (sh.red[slot][2][s][1] + sh.red[slot][3][s][1]);
    }
    slot ^= 1;
}

template <int METHOD, int CTRL>
__global__ void __launch_bounds__(256) solve_mlp_kernel(const SolveParams<float> p, const float *weights, const MlpOut o) {
    using T = float;
    using Tab = typename std::conditional<METHOD == 1, Tsit5Tab, Dopri5Tab>::type;
    constexpr int F = MLP_F, H = MLP_H;
    __shared__ MlpShared sh;
    extern __shared__ __align__(16) unsigned char dyn[];
    T *te_s = reinterpret_cast<T *>(dyn);  // [16][E]

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, q = lane >> 4, c = lane & 15;
    const long long b0 = (long long)blockIdx.x * MLP_TILE;
    const int rows = (int)min((long long)MLP_TILE, p.batch - b0);
    const int E = p.n_eval;
    const CtrlParams<T> &cp = p.cp;
    const T sf = (T)__builtin_sqrt((double)F);
    const int f = 16 * w + c;
    int slot = 0;

    // ---- weights into registers: [W1 (H x 65) | b1 (H) | W2 (F x H) | b2 (F)] ----
    MlpWeights W;
    {
        const float *W1 = weights, *b1 = W1 + H * (F + 1), *W2 = b1 + H, *b2 = W2 + F * H;
#pragma unroll
        for (int kk = 0; kk < 17; ++kk)
#pragma unroll
            for (int tile = 0; tile < 4; ++tile) {
                const int k = 4 * kk + q;
                W.w1[kk][tile] = k <= F ? W1[(64 * w + 16 * tile + c) * (F + 1) + k] : 0.0f;
            }
#pragma unroll
        for (int tile = 0; tile < 4; ++tile) W.b1[tile] = b1[64 * w + 16 * tile + c];
#pragma unroll
        for (int kk = 0; kk < 64; ++kk) W.w2[kk] = W2[f * H + 4 * kk + q];
        W.b2 = b2[f];
    }
    for (int i = tid; i < MLP_TILE * MLP_XS; i += 256) sh.x[i] = 0.0f;  // also the padding columns 65..67
    for (int i = tid; i < rows * E; i += 256) te_s[i] = p.t_eval[b0 * E + i];
    __syncthreads();

    // ---- per-sample state of the lane's four samples ----
    bool live[4], active[4], bail = false;
    long long bs[4];
    T ts[4], te[4], dir[4], tlo[4], thi[4], t[4], dt[4], y[4], k[7][4], prev[4], pprev[4];
    int cursor[4], n_steps[4], n_acc[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int s = 4 * q + r;
        live[r] = s < rows;
        bs[r] = b0 + (live[r] ? s : 0);
        ts[r] = p.t_start[bs[r] * p.ts_stride];
        te[r] = p.t_end[bs[r] * p.te_stride];
        dir[r] = (te[r] > ts[r]) ? (T)1 : (T)-1;
        tlo[r] = tmin(ts[r], te[r]);
        thi[r] = tmax(te[r], ts[r]);
        y[r] = p.y0[bs[r] * F + f];
        t[r] = ts[r];
        prev[r] = pprev[r] = 1;
        cursor[r] = n_steps[r] = n_acc[r] = 0;
        const T *tev = te_s + (live[r] ? s : 0) * E;
        for (int e = 1; e < E; ++e) bail = bail || (live[r] && !(dir[r] * tev[e] >= dir[r] * tev[e - 1]));  // not monotone
    }

    // ---- first step size (step_size_controllers.py:431-490, 776-835) ----
    mlp_rhs(sh, W, ts, y, k[0]);
    if (p.dt0) {
#pragma unroll
        for (int r = 0; r < 4; ++r) dt[r] = p.dt0[bs[r]];
    } else {
        T inv[4], a0[4], a1[4], A0[4], A1[4], h0[4], y1[4], t1[4], f1[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            inv[r] = inv_scale(cp.atol, cp.rtol, y[r]);
            const T x0 = (y[r] * inv[r]) / sf, x1 = (k[0][r] * inv[r]) / sf;
            a0[r] = x0 * x0;
            a1[r] = x1 * x1;
        }
        mlp_sum2(sh, slot, a0, a1, A0, A1);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const T d0 = sqrt_(A0[r]), d1 = sqrt_(A1[r]);
            T h = (d0 < (T)1e-5 || d1 < (T)1e-5) ? (T)1e-6 : ((T)0.01 * d0) / d1;
            h0[r] = tmin(h, abs_(te[r] - ts[r]));
            y1[r] = fma_(dir[r] * h0[r], k[0][r], y[r]);
            t1[r] = fma_(dir[r], h0[r], ts[r]);
        }
        mlp_rhs(sh, W, t1, y1, f1);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const T df = f1[r] - k[0][r];
            const T x2 = (df * inv[r]) / sf;
            a0[r] = x2 * x2;
        }
        T A2[4];
        mlp_sum2(sh, slot, a0, a1, A2, A1);  // A1 (the norm of f0) comes out again unchanged
#pragma unroll
        for (int r = 0; r < 4; ++r)
            dt[r] = initial_finish<T>(CTRL == 1 ? TODE_CTRL_PID : TODE_CTRL_INTEGRAL, 1.0 / 5.0, dir[r], h0[r], sqrt_(A1[r]), sqrt_(A2[r]));
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        dt[r] = tclamp(dt[r], tlo[r] - t[r], thi[r] - t[r]);
        active[r] = live[r];
        if (live[r] && E > 0 && te_s[(4 * q + r) * E] == ts[r]) {
            p.ys[(bs[r] * E) * F + f] = y[r];
            cursor[r] = 1;
        }
    }
    bail = __syncthreads_or(bail) != 0;

    while (!bail && __syncthreads_or(active[0] || active[1] || active[2] || active[3])) {
        // ---- stages (runge_kutta.py:255-263) ----
        T t0[4], y1[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) t0[r] = t[r];
#pragma unroll
        for (int i = 1; i < 7; ++i) {
            T tn[4], yi[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                tn[r] = fma_((T)Tab::c[i], dt[r], t0[r]);
                T s = 0;
#pragma unroll
                for (int j = 0; j < i; ++j) s = fma_((T)Tab::a[i][j], k[j][r], s);
                yi[r] = fma_(dt[r], s, y[r]);
            }
            mlp_rhs(sh, W, tn, yi, k[i]);
            if (i == 6) {
#pragma unroll
                for (int r = 0; r < 4; ++r) y1[r] = yi[r];
            }
        }

        // ---- error ratio (runge_kutta.py:267, step_size_controllers.py:389-395); F >= 58: fused sums ----
        T part[4], zero[4] = {0, 0, 0, 0}, total[4], unused[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            T err = 0;
#pragma unroll
            for (int s = 0; s < 7; ++s) err = fma_(dt[r] * (T)Tab::b_err[s], k[s][r], err);
            const T m = tmax(abs_(y[r]), abs_(y1[r]));
            const T x = (abs_(err) / fma_(cp.rtol, m, cp.atol)) / sf;
            part[r] = x * x;
        }
        mlp_sum2(sh, slot, part, zero, total, unused);

#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const T ratio = tmax(sqrt_(total[r]), (T)1e-38);
            const bool accept = ratio < (T)1;
            T dt_next = dt[r] * dt_factor<T, CTRL>(cp, ratio, prev[r], pprev[r]);
            const int status = limit_dt<T>(cp, ratio, dt_next);
            const bool move = accept && active[r];
            const T t_new = move ? (t0[r] + dt[r]) : t0[r];
            const bool running_new = fma_(dir[r], t_new, -dir[r] * te[r]) < (T)0;
            n_steps[r] += active[r] ? 1 : 0;
            n_acc[r] += move ? 1 : 0;

            // ---- dense output at the evaluation points this step passed (adjoints.py:215-234) ----
            const T *tev = te_s + (live[r] ? 4 * q + r : 0) * E;
            if (active[r] && cursor[r] < E && fma_(dir[r], t_new, -dir[r] * tev[cursor[r]]) >= (T)0) {
                T ks[7], qc[5][1];
#pragma unroll
                for (int s = 0; s < 7; ++s) ks[s] = k[s][r];
                quartic_elem<T, METHOD>(dt[r], y[r], y1[r], ks, true, qc);
                const T t1 = t0[r] + dt[r];
                do {
                    const T x = unit_time(tev[cursor[r]], t0[r], t1);
                    T v = qc[4][0];
#pragma unroll
                    for (int pw = 3; pw >= 0; --pw) v = fma_(v, x, qc[pw][0]);
                    p.ys[(bs[r] * E + cursor[r]) * F + f] = v;
                    ++cursor[r];
                } while (cursor[r] < E && fma_(dir[r], t_new, -dir[r] * tev[cursor[r]]) >= (T)0);
            }

            // ---- state update (adjoints.py:150-155, 247-255) ----
            y[r] = move ? y1[r] : y[r];
            k[0][r] = move ? k[6][r] : k[0][r];
            t[r] = t_new;
            const T dtc = tclamp(running_new ? dt_next : dt[r], tlo[r] - t_new, thi[r] - t_new);
            dt[r] = active[r] ? dtc : dt[r];
            if (CTRL == 1 && active[r] && running_new && accept) {
                pprev[r] = prev[r];
                prev[r] = ratio;
            }
            const bool failed = active[r] && (status != 0 || n_steps[r] >= p.max_steps || n_steps[r] >= TODE_HARD_STEP_LIMIT);
            const bool finished = active[r] && !failed && !running_new;
            // a sample that does not land on t_end, or ends on a non-finite value, shows up in later
            // iterations of the reference loop: not the common case
            const bool odd = !(t[r] == te[r]) || !finite_(y[r]) || !finite_(k[0][r]);
            bail = bail || failed || (finished && odd);
            active[r] = active[r] && !failed && running_new;
        }
        bail = __syncthreads_or(bail) != 0;
    }

    if (w == 0 && c == 0) {
        int most = 0;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            if (!live[r]) continue;
            o.n_steps[bs[r]] = n_steps[r];
            o.n_accepted[bs[r]] = n_acc[r];
            o.n_initialized[bs[r]] = cursor[r];
            o.status[bs[r]] = 0;
            most = max(most, n_steps[r]);
        }
        if (most > 0) atomicMax(&p.flags[TODE_FLAG_MAX_ITERATIONS], most);
        if (bail) atomicMax(&p.flags[TODE_FLAG_NEEDS_GENERAL], 1);
    }
    publish_flags(p);
}

template <int METHOD, int CTRL> static int launch_mlp(const tode_solve_args &a, const tode_controller &c, const MlpOut &o, hipStream_t stream) {
    SolveParams<float> p = make_params<float>(a, c);
    reset_flags(a.flags, stream);
    if (a.batch == 0) return check_hip(hipGetLastError(), "tode_solve_builtin_fast launch");
    const size_t lds = (size_t)MLP_TILE * a.n_eval * sizeof(float);
    const unsigned blocks = (unsigned)((a.batch + MLP_TILE - 1) / MLP_TILE);
    timing_before(stream, "tode::solve_mlp_kernel");
    hipLaunchKernelGGL((solve_mlp_kernel<METHOD, CTRL>), dim3(blocks), dim3(256), lds, stream, p, (const float *)a.shared_params, o);
    timing_after(stream);
    return check_hip(hipGetLastError(), "tode_solve_builtin_fast launch");
}

int solve_mlp_f32(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s) {
    const long long need = (long long)MLP_H * (MLP_F + 1) + MLP_H + (long long)MLP_F * MLP_H + MLP_F;
    if (a.n_features != MLP_F || a.n_shared_params != need)
        return fail(TODE_E_UNSUPPORTED, "the MLP kernel is built for 64 features and 256 hidden units (%lld shared parameters), got F=%d and %lld",
                    need, a.n_features, (long long)a.n_shared_params);
    if (!a.shared_params) return fail(TODE_E_INVALID, "null shared_params");
    if (a.n_eval > 512) return fail(TODE_E_UNSUPPORTED, "n_eval=%d is too large for the MLP kernel", a.n_eval);
    if (a.batch > (long long)INT_MAX * MLP_TILE) return fail(TODE_E_UNSUPPORTED, "batch too large");
    MlpOut o{ns, na, ni, st};
    if (a.method == TODE_DOPRI5 && c.kind == TODE_CTRL_INTEGRAL) return launch_mlp<0, 0>(a, c, o, s);
    if (a.method == TODE_DOPRI5 && c.kind == TODE_CTRL_PID) return launch_mlp<0, 1>(a, c, o, s);
    if (a.method == TODE_TSIT5 && c.kind == TODE_CTRL_INTEGRAL) return launch_mlp<1, 0>(a, c, o, s);
    if (a.method == TODE_TSIT5 && c.kind == TODE_CTRL_PID) return launch_mlp<1, 1>(a, c, o, s);
    return fail(TODE_E_INVALID, "unknown method %d or controller kind %d", a.method, c.kind);
}

}  // namespace tode
