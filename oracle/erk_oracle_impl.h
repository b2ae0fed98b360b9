/*
 * TEST INFRASTRUCTURE ONLY -- body of the scalar CPU oracle, included once per
 * floating point type by erk_oracle.c (REAL, SFX, and the R_* helpers are
 * defined there).  See erk_oracle.c for the provenance of every function.
 */

/* ---- NaN-propagating min / max / clamp (torch.maximum, torch.minimum, torch.clamp) ---- */
static inline REAL SFX(tmax)(REAL a, REAL b) { return (a != a) ? a : ((b != b) ? b : (a > b ? a : b)); }
static inline REAL SFX(tmin)(REAL a, REAL b) { return (a != a) ? a : ((b != b) ? b : (a < b ? a : b)); }
static inline REAL SFX(tclamp)(REAL x, REAL lo, REAL hi) { return SFX(tmin)(SFX(tmax)(x, lo), hi); }

/* tensor ** python_float as ATen's CPU kernels compute it: exponents 0 and 1 are a fill and a copy
 * (aten/src/ATen/native/Pow.cpp), 0.5, -0.5 and -1 go to the square root, reciprocal square root and reciprocal kernels,
 * 2, 3 and -2 are multiplications (aten/src/ATen/native/cpu/PowKernel.cpp); every other exponent is rounded to the
 * tensor dtype and goes through pow.  The first group compares the exponent as the double it is, the second after
 * rounding to the tensor dtype.  The square roots here are the correctly rounded ones; an ATen build that takes them
 * from a vector math library can differ from that in the last bit (exponents 0.5 and -0.5 only). */
static inline REAL SFX(rpow)(REAL x, double p) {
    if (p == 0.0) return (REAL)1;
    if (p == 1.0) return x;
    if (p == 0.5) return R_SQRT(x);
    if (p == -0.5) return (REAL)1 / R_SQRT(x);
    if (p == -1.0) return (REAL)1 / x;
    REAL e = (REAL)p;
    if (e == (REAL)2) return x * x;
    if (e == (REAL)3) return (x * x) * x;
    if (e == (REAL)-2) return (REAL)1 / (x * x);
    return R_POW(x, e);
}

/* ---- built-in right-hand sides, canonical op order, every op rounded on its own ---- */
static void SFX(rhs)(const oracle_config *cfg, const REAL *par, REAL t, const REAL *y, REAL *dy, int F) {
    (void)t;
    switch (cfg->term) {
    case ORACLE_TERM_LINEAR_DECAY: /* (-k) * y */
        for (int f = 0; f < F; ++f) dy[f] = (-par[f]) * y[f];
        break;
    case ORACLE_TERM_VDP: { /* dx = v ; dv = ((mu*(1-(x*x)))*v)-x */
        REAL x = y[0], v = y[1], mu = par[0];
        REAL xx = x * x;
        REAL om = (REAL)1 - xx;
        REAL m1 = mu * om;
        REAL m2 = m1 * v;
        dy[0] = v;
        dy[1] = m2 - x;
        break;
    }
    case ORACLE_TERM_LORENZ: { /* dx=sigma*(y-x); dy=(x*(rho-z))-y; dz=(x*y)-(beta*z) */
        REAL x = y[0], yy = y[1], z = y[2], rho = par[0];
        REAL sigma = (REAL)10.0, beta = (REAL)(8.0 / 3.0);
        REAL d1 = yy - x;
        REAL r1 = rho - z;
        REAL xr = x * r1;
        REAL xy = x * yy;
        REAL bz = beta * z;
        dy[0] = sigma * d1;
        dy[1] = xr - yy;
        dy[2] = xy - bz;
        break;
    }
    default:
        for (int f = 0; f < F; ++f) dy[f] = (REAL)NAN;
    }
}

/* rms_norm(v): sqrt(sum_f (v_f / sqrt(F))^2), step_size_controllers.py:170-181.
 * Association observed for ATen's CPU vector_norm over the inner dimension:
 * F <= 3 a fused chain acc = fma(x,x,acc), F >= 4 acc = acc + x*x with the
 * product rounded first. */
static REAL SFX(rms)(const REAL *v, int F) {
    REAL sf = (REAL)sqrt((double)F);
    REAL acc = 0;
    for (int f = 0; f < F; ++f) {
        REAL x = v[f] / sf;
        if (F <= 3)
            acc = R_FMA(x, x, acc);
        else {
            REAL sq = x * x;
            acc = acc + sq;
        }
    }
    return R_SQRT(acc);
}

/* sum_s round(dt*w_s) * k_s : einsum("b, s, sbf -> bf").  F <= 57 products are
 * rounded before they are added, F >= 58 a fused chain (ATen bmm small-matrix
 * path versus gemm). */
static void SFX(weighted_k)(REAL dt, const double *w, const REAL *k, int S, int F, REAL *out) {
    for (int f = 0; f < F; ++f) {
        REAL acc = 0;
        for (int s = 0; s < S; ++s) {
            REAL p = dt * (REAL)w[s];
            if (F <= 57) {
                REAL pk = p * k[s * F + f];
                acc = acc + pk;
            } else
                acc = R_FMA(p, k[s * F + f], acc);
        }
        out[f] = acc;
    }
}

/* One FSAL+SSAL explicit RK step, runge_kutta.py:247-272.  k is [7][F] with
 * k[0] already holding the FSAL derivative. */
static void SFX(erk_step)(const oracle_config *cfg, const oracle_tableau *tab, const REAL *par, REAL t0, REAL dt,
                          const REAL *y0, REAL *k, REAL *y1, REAL *err, REAL *ytmp, int F) {
    for (int i = 1; i < 7; ++i) {
        REAL tn = R_FMA((REAL)tab->c[i], dt, t0);
        for (int f = 0; f < F; ++f) {
            REAL s = 0;
            for (int j = 0; j < i; ++j) s = R_FMA((REAL)tab->a[i][j], k[j * F + f], s);
            ytmp[f] = R_FMA(dt, s, y0[f]);
        }
        SFX(rhs)(cfg, par, tn, ytmp, k + i * F, F);
        if (i == 6)
            for (int f = 0; f < F; ++f) y1[f] = ytmp[f];
    }
    SFX(weighted_k)(dt, tab->b_err, k, 7, F, err);
}

/* Error ratio (step_size_controllers.py:393-401 / 738-746). */
static REAL SFX(error_ratio)(const oracle_config *cfg, const REAL *y0, const REAL *y1, const REAL *err, REAL *tmp, int F) {
    REAL atol = (REAL)(float)cfg->atol, rtol = (REAL)(float)cfg->rtol;
    for (int f = 0; f < F; ++f) {
        REAL m = SFX(tmax)(R_ABS(y0[f]), R_ABS(y1[f]));
        REAL eb = R_FMA(rtol, m, atol);
        tmp[f] = R_ABS(err[f]) / eb;
    }
    return SFX(tmax)(SFX(rms)(tmp, F), (REAL)1e-38);
}

/* dt factor (step_size_controllers.py:289-294, 598-620). */
static REAL SFX(dt_factor)(const oracle_config *cfg, REAL ratio, REAL prev, REAL prev_prev) {
    double order = 5.0;
    REAL factor;
    if (cfg->controller == ORACLE_CTRL_INTEGRAL) {
        double k_i = 1.0 / order;
        factor = (REAL)cfg->safety * SFX(rpow)(ratio, -k_i);
    } else {
        double k_i = cfg->icoeff / order, k_p = cfg->pcoeff / order, k_d = cfg->dcoeff / order;
        REAL f1 = SFX(rpow)(ratio, -(k_i + k_p + k_d));
        REAL f2 = SFX(rpow)(prev, k_p + 2 * k_d);
        REAL f3 = SFX(rpow)(prev_prev, -k_d);
        factor = (REAL)cfg->safety * f1;
        factor = factor * f2;
        factor = factor * f3;
    }
    return SFX(tclamp)(factor, (REAL)cfg->factor_min, (REAL)cfg->factor_max);
}

/* Start step (step_size_controllers.py:431-490 integral, 776-835 PID). */
static REAL SFX(initial_step)(const oracle_config *cfg, const REAL *par, REAL t0, const REAL *y0, REAL dir, REAL span,
                              REAL *f0, REAL *w1, REAL *w2, REAL *w3, int F) {
    REAL atol = (REAL)(float)cfg->atol, rtol = (REAL)(float)cfg->rtol;
    SFX(rhs)(cfg, par, t0, y0, f0, F);
    REAL *inv = w1;
    for (int f = 0; f < F; ++f) inv[f] = (REAL)1 / R_FMA(rtol, R_ABS(y0[f]), atol);
    for (int f = 0; f < F; ++f) w2[f] = y0[f] * inv[f];
    REAL d0 = SFX(rms)(w2, F);
    for (int f = 0; f < F; ++f) w2[f] = f0[f] * inv[f];
    REAL d1 = SFX(rms)(w2, F);
    REAL tiny = (REAL)1e-6;
    REAL h0 = (d0 < (REAL)1e-5 || d1 < (REAL)1e-5) ? tiny : ((REAL)0.01 * d0) / d1;
    h0 = SFX(tmin)(h0, span);
    REAL dh = dir * h0;
    for (int f = 0; f < F; ++f) w2[f] = R_FMA(dh, f0[f], y0[f]);
    REAL t1 = R_FMA(dir, h0, t0);
    SFX(rhs)(cfg, par, t1, w2, w3, F);
    for (int f = 0; f < F; ++f) {
        REAL df = w3[f] - f0[f];
        w2[f] = df * inv[f];
    }
    REAL d2 = SFX(rms)(w2, F) / h0;
    if (cfg->controller == ORACLE_CTRL_INTEGRAL && h0 == 0) d2 = (REAL)INFINITY;
    REAL m = SFX(tmax)(d1, d2);
    REAL h1;
    if (m <= (REAL)1e-15)
        h1 = SFX(tmax)(tiny, h0 * (REAL)1e-3);
    else {
        /* `0.01 / tensor` is evaluated by torch as reciprocal(tensor) * 0.01 */
        REAL rm = (REAL)1 / m;
        h1 = SFX(rpow)(rm * (REAL)0.01, 1.0 / 5.0);
    }
    return dir * SFX(tmin)((REAL)100 * h0, h1);
}

/* Quartic coefficients, lowest power first in q[5][F]
 * (tsit5.py:123-139; dopri5.py:53-60 -> interpolation.py:138-170). */
static void SFX(quartic)(const oracle_config *cfg, const oracle_tableau *tab, REAL dt, const REAL *y0, const REAL *y1,
                         const REAL *k, REAL *q, int F) {
    if (cfg->method == ORACLE_METHOD_TSIT5) {
        for (int f = 0; f < F; ++f) {
            q[0 * F + f] = y0[f];
            q[1 * F + f] = dt * k[f];
        }
        for (int p = 0; p < 3; ++p) SFX(weighted_k)(dt, tab->b_other[p], k, 7, F, q + (2 + p) * F);
    } else {
        REAL *ymid = q + 2 * F; /* scratch, overwritten last */
        SFX(weighted_k)(dt, tab->b_other[0], k, 7, F, ymid);
        for (int f = 0; f < F; ++f) {
            REAL f0 = dt * k[f], f1 = dt * k[6 * F + f];
            REAL ym = y0[f] + ymid[f];
            REAL df = f1 - f0;
            REAL sy = y1[f] + y0[f];
            REAL a = (REAL)2 * df;
            a = R_FMA((REAL)-8, sy, a);
            a = R_FMA((REAL)16, ym, a);
            REAL b = (REAL)5 * f0;
            b = R_FMA((REAL)-3, f1, b);
            b = R_FMA((REAL)18, y0[f], b);
            b = R_FMA((REAL)14, y1[f], b);
            b = R_FMA((REAL)-32, ym, b);
            REAL c = R_FMA((REAL)-4, f0, f1);
            c = R_FMA((REAL)-11, y0[f], c);
            c = R_FMA((REAL)-5, y1[f], c);
            c = R_FMA((REAL)16, ym, c);
            q[0 * F + f] = y0[f];
            q[1 * F + f] = f0;
            q[2 * F + f] = c;
            q[3 * F + f] = b;
            q[4 * F + f] = a;
        }
    }
}

/* Horner on x = (t - t0) / (t1 - t0), interpolation.py:25-40. */
static void SFX(quartic_eval)(const REAL *q, REAL t0, REAL dt, REAL t, REAL *out, int F) {
    REAL t1 = t0 + dt;
    REAL den = t1 - t0;
    if (!(R_ABS(den) > (REAL)0)) den = (REAL)1;
    REAL x = (t - t0) / den;
    for (int f = 0; f < F; ++f) {
        REAL y = q[4 * F + f];
        y = R_FMA(y, x, q[3 * F + f]);
        y = R_FMA(y, x, q[2 * F + f]);
        y = R_FMA(y, x, q[1 * F + f]);
        y = R_FMA(y, x, q[0 * F + f]);
        out[f] = y;
    }
}

/* ---- single-function entry points used by the pin tests ---- */

void SFX(oracle_rhs)(const oracle_config *cfg, const REAL *par, REAL t, const REAL *y, REAL *dy, int F) {
    SFX(rhs)(cfg, par, t, y, dy, F);
}

void SFX(oracle_erk_step)(const oracle_config *cfg, const REAL *par, REAL t0, REAL dt, const REAL *y0, const REAL *k0,
                          REAL *k, REAL *y1, REAL *err, int F) {
    REAL *tmp = (REAL *)malloc(sizeof(REAL) * F);
    for (int f = 0; f < F; ++f) k[f] = k0[f];
    SFX(erk_step)(cfg, oracle_get_tableau(cfg->method), par, t0, dt, y0, k, y1, err, tmp, F);
    free(tmp);
}

/* out = {ratio, accept, dt_next, status, prev_new, prev_prev_new} */
void SFX(oracle_adapt)(const oracle_config *cfg, REAL dt, const REAL *y0, const REAL *y1, const REAL *err, REAL prev,
                       REAL prev_prev, REAL *out, int F) {
    REAL *tmp = (REAL *)malloc(sizeof(REAL) * F);
    REAL ratio = SFX(error_ratio)(cfg, y0, y1, err, tmp, F);
    free(tmp);
    int accept = ratio < (REAL)1;
    REAL dt_next = dt * SFX(dt_factor)(cfg, ratio, prev, prev_prev);
    int status = R_ISFINITE(ratio) ? ORACLE_SUCCESS : ORACLE_INFINITE_NORM;
    if (cfg->has_dt_min || cfg->has_dt_max) {
        REAL mag = R_ABS(dt_next);
        REAL c = mag;
        if (cfg->has_dt_min) c = SFX(tmax)(c, (REAL)cfg->dt_min);
        if (cfg->has_dt_max) c = SFX(tmin)(c, (REAL)cfg->dt_max);
        REAL sg = (dt_next > 0) ? (REAL)1 : ((dt_next < 0) ? (REAL)-1 : dt_next /* 0 or NaN */);
        dt_next = sg * c;
        if (cfg->has_dt_min && mag < (REAL)cfg->dt_min) status = ORACLE_REACHED_DT_MIN;
    }
    out[0] = ratio;
    out[1] = (REAL)accept;
    out[2] = dt_next;
    out[3] = (REAL)status;
    if (cfg->controller == ORACLE_CTRL_PID) {
        out[4] = accept ? ratio : prev;
        out[5] = accept ? prev : prev_prev;
    } else {
        out[4] = prev;
        out[5] = prev_prev;
    }
}

REAL SFX(oracle_initial_step)(const oracle_config *cfg, const REAL *par, REAL t0, const REAL *y0, REAL t_end, REAL *f0,
                              int F) {
    REAL *w = (REAL *)malloc(sizeof(REAL) * 3 * F);
    REAL dir = (t_end > t0) ? (REAL)1 : (REAL)-1;
    REAL r = SFX(initial_step)(cfg, par, t0, y0, dir, R_ABS(t_end - t0), f0, w, w + F, w + 2 * F, F);
    free(w);
    return r;
}

void SFX(oracle_quartic)(const oracle_config *cfg, REAL dt, const REAL *y0, const REAL *y1, const REAL *k, REAL *q, int F) {
    SFX(quartic)(cfg, oracle_get_tableau(cfg->method), dt, y0, y1, k, q, F);
}

void SFX(oracle_quartic_eval)(const REAL *q, REAL t0, REAL dt, REAL t, REAL *out, int F) {
    SFX(quartic_eval)(q, t0, dt, t, out, F);
}

/* ---- the lock-step solve loop, adjoints.py:50-309 ---- */

typedef struct {
    REAL t, dt, prev, prev_prev;
    int running;
    int status;
} SFX(sample_state);

int SFX(oracle_solve)(const oracle_config *cfg, int64_t B, int F, int E, const REAL *y0_in, const REAL *t_start,
                      const REAL *t_end, const REAL *t_eval, const REAL *dt0, const REAL *params, int P, REAL *ys,
                      int64_t *n_steps, int64_t *n_accepted, int64_t *n_initialized, int64_t *status_out,
                      int64_t *n_f_evals, REAL *trace, int64_t trace_iters, int64_t trace_B, unsigned char *written) {
    const oracle_tableau *tab = oracle_get_tableau(cfg->method);
    if (!tab) return -1;
    int nthreads = cfg->nthreads > 0 ? cfg->nthreads : 1;
    SFX(sample_state) *st = (SFX(sample_state) *)calloc((size_t)B, sizeof(*st));
    REAL *y = (REAL *)malloc(sizeof(REAL) * (size_t)B * F);
    REAL *k0 = (REAL *)malloc(sizeof(REAL) * (size_t)B * F);
    unsigned char *pending = (unsigned char *)malloc((size_t)B * (E > 0 ? E : 1));
    /* per-thread workspaces: k[7F], y1, err, tmp, q[5F], out */
    size_t wsz = (size_t)(7 + 1 + 1 + 1 + 5 + 1 + 3) * F;
    REAL *work = (REAL *)malloc(sizeof(REAL) * wsz * nthreads);
    int64_t evals = 0;

    /* init: start step (2 f evaluations) or user dt0 (1 evaluation for the FSAL slot) */
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t b = 0; b < B; ++b) {
#ifdef _OPENMP
        REAL *w = work + wsz * omp_get_thread_num();
#else
        REAL *w = work;
#endif
        const REAL *par = params + (size_t)b * P;
        REAL dir = (t_end[b] > t_start[b]) ? (REAL)1 : (REAL)-1;
        for (int f = 0; f < F; ++f) y[b * F + f] = y0_in[b * F + f];
        REAL dt;
        if (dt0)  {
            dt = dt0[b];
            SFX(rhs)(cfg, par, t_start[b], y + b * F, k0 + b * F, F);
        } else {
            dt = SFX(initial_step)(cfg, par, t_start[b], y + b * F, dir, R_ABS(t_end[b] - t_start[b]), k0 + b * F, w, w + F,
                                   w + 2 * F, F);
        }
        REAL tmin = SFX(tmin)(t_start[b], t_end[b]), tmax = SFX(tmax)(t_end[b], t_start[b]);
        st[b].t = t_start[b];
        st[b].dt = SFX(tclamp)(dt, tmin - st[b].t, tmax - st[b].t);
        st[b].prev = st[b].prev_prev = (REAL)1;
        st[b].running = 1;
        st[b].status = ORACLE_SUCCESS;
        n_steps[b] = 0;
        n_accepted[b] = 0;
        for (int e = 0; e < E; ++e) pending[b * E + e] = 1;
        if (t_eval && E > 0 && t_eval[b * E] == t_start[b]) {
            for (int f = 0; f < F; ++f) ys[((size_t)b * E) * F + f] = y[b * F + f];
            pending[b * E] = 0;
        }
    }
    evals += dt0 ? 1 : 2;

    int64_t it = 0;
    for (;;) {
        int any_running = 0, all_success = 1;
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 64) reduction(| : any_running) reduction(& : all_success)
        for (int64_t b = 0; b < B; ++b) {
#ifdef _OPENMP
            REAL *w = work + wsz * omp_get_thread_num();
#else
            REAL *w = work;
#endif
            REAL *k = w, *y1 = w + 7 * F, *err = w + 8 * F, *tmp = w + 9 * F, *q = w + 10 * F, *out = w + 15 * F;
            const REAL *par = params + (size_t)b * P;
            SFX(sample_state) *s = &st[b];
            REAL dir = (t_end[b] > t_start[b]) ? (REAL)1 : (REAL)-1;
            REAL *yb = y + b * F;
            for (int f = 0; f < F; ++f) k[f] = k0[b * F + f];
            REAL t0 = s->t, dt = s->dt;
            SFX(erk_step)(cfg, tab, par, t0, dt, yb, k, y1, err, tmp, F);

            REAL ratio = SFX(error_ratio)(cfg, yb, y1, err, tmp, F);
            int accept = ratio < (REAL)1;
            REAL dt_next = dt * SFX(dt_factor)(cfg, ratio, s->prev, s->prev_prev);
            int status = R_ISFINITE(ratio) ? ORACLE_SUCCESS : ORACLE_INFINITE_NORM;
            if (cfg->has_dt_min || cfg->has_dt_max) {
                REAL mag = R_ABS(dt_next);
                REAL c = mag;
                if (cfg->has_dt_min) c = SFX(tmax)(c, (REAL)cfg->dt_min);
                if (cfg->has_dt_max) c = SFX(tmin)(c, (REAL)cfg->dt_max);
                REAL sg = (dt_next > 0) ? (REAL)1 : ((dt_next < 0) ? (REAL)-1 : dt_next);
                dt_next = sg * c;
                if (cfg->has_dt_min && mag < (REAL)cfg->dt_min) status = ORACLE_REACHED_DT_MIN;
            }
            REAL prev_n = s->prev, pprev_n = s->prev_prev;
            if (cfg->controller == ORACLE_CTRL_PID && accept) {
                prev_n = ratio;
                pprev_n = s->prev;
            }
            if (trace && it < trace_iters && b < trace_B) {
                REAL *tr = trace + ((size_t)it * trace_B + b) * 4;
                tr[0] = t0;
                tr[1] = dt;
                tr[2] = ratio;
                tr[3] = (REAL)(accept + 2 * s->running);
            }

            /* quartic of the attempted step is built from the pre-update state */
            int need_interp = 0;
            int move = accept && s->running;
            REAL t_new = move ? (t0 + dt) : t0;
            if (t_eval) {
                for (int e = 0; e < E; ++e) {
                    if (!pending[b * E + e]) continue;
                    /* addcmul(-dir*t_eval, dir, t) >= 0 */
                    REAL v = R_FMA(dir, t_new, -dir * t_eval[b * E + e]);
                    if (v >= (REAL)0) {
                        if (!need_interp) {
                            SFX(quartic)(cfg, tab, dt, yb, y1, k, q, F);
                            need_interp = 1;
                        }
                        SFX(quartic_eval)(q, t0, dt, t_eval[b * E + e], out, F);
                        for (int f = 0; f < F; ++f) ys[((size_t)b * E + e) * F + f] = out[f];
                        pending[b * E + e] = 0;
                    }
                }
            }

            /* t_eval == NULL (adjoints.py:295-309): the interpolant of the last iteration is
             * evaluated at t_end; overwriting the slot every iteration leaves exactly that. */
            if (!t_eval) {
                SFX(quartic)(cfg, tab, dt, yb, y1, k, q, F);
                SFX(quartic_eval)(q, t0, dt, t_end[b], out, F);
                for (int f = 0; f < F; ++f) ys[(size_t)b * F + f] = out[f];
            }

            n_steps[b] += s->running;
            n_accepted[b] += move;
            if (move) {
                for (int f = 0; f < F; ++f) {
                    yb[f] = y1[f];
                    k0[b * F + f] = k[6 * F + f];
                }
            }
            s->t = t_new;
            int running_new = R_FMA(dir, t_new, -dir * t_end[b]) < (REAL)0;
            if (cfg->max_steps >= 0 && n_steps[b] >= cfg->max_steps) status = ORACLE_REACHED_MAX_STEPS;
            s->status = status;

            REAL dtn = running_new ? dt_next : dt;
            REAL tmin = SFX(tmin)(t_start[b], t_end[b]), tmax = SFX(tmax)(t_end[b], t_start[b]);
            s->dt = SFX(tclamp)(dtn, tmin - t_new, tmax - t_new);
            if (running_new) {
                s->prev = prev_n;
                s->prev_prev = pprev_n;
            }
            s->running = running_new;
            any_running |= running_new;
            all_success &= (status == ORACLE_SUCCESS);
        }
        evals += 6;
        ++it;
        if (any_running && all_success) continue;
        break;
    }

    for (int64_t b = 0; b < B; ++b) {
        status_out[b] = st[b].status;
        if (t_eval) {
            /* adjoints.py:289-292: torch.searchsorted(not_yet_evaluated.int(), 1), i.e. ATen's lower-bound binary
               search -- the index of the first pending point when the row of marks is sorted (evaluation times
               monotone in the sample's direction), and whatever the search lands on when it is not */
            int64_t lo = 0, hi = E;
            while (lo < hi) {
                const int64_t mid = lo + ((hi - lo) >> 1);
                if (!pending[b * E + mid]) lo = mid + 1; else hi = mid;
            }
            n_initialized[b] = lo;
        } else {
            n_initialized[b] = 1;
        }
    }
    *n_f_evals = evals;
    free(st);
    free(y);
    free(k0);
    if (written)
        for (int64_t i = 0; i < B * (int64_t)E; ++i) written[i] = !pending[i];
    free(pending);
    free(work);
    return 0;
}
