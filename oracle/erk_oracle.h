/* TEST INFRASTRUCTURE ONLY -- declarations of the scalar CPU oracle (erk_oracle.c). */
#ifndef ERK_ORACLE_H
#define ERK_ORACLE_H
#include <stdint.h>

enum { ORACLE_METHOD_DOPRI5 = 0, ORACLE_METHOD_TSIT5 = 1 };
enum { ORACLE_CTRL_INTEGRAL = 0, ORACLE_CTRL_PID = 1 };
enum { ORACLE_TERM_LINEAR_DECAY = 0, ORACLE_TERM_VDP = 1, ORACLE_TERM_LORENZ = 2 };
enum {
    ORACLE_SUCCESS = 0,
    ORACLE_GENERAL_ERROR = 1,
    ORACLE_REACHED_DT_MIN = 2,
    ORACLE_REACHED_MAX_STEPS = 3,
    ORACLE_INFINITE_NORM = 4
};

typedef struct {
    double c[7];
    double a[7][7];
    double b[7];
    double b_err[7];
    double b_other[3][7];
    int n_other;
} oracle_tableau;

typedef struct {
    int32_t method;     /* ORACLE_METHOD_*  */
    int32_t controller; /* ORACLE_CTRL_*    */
    int32_t term;       /* ORACLE_TERM_*    */
    int32_t nthreads;   /* OpenMP threads over samples, >= 1 */
    double atol, rtol;  /* rounded to float32 inside, as the reference stores them */
    double pcoeff, icoeff, dcoeff;
    double safety, factor_min, factor_max;
    int32_t has_dt_min, has_dt_max;
    double dt_min, dt_max;
    int64_t max_steps; /* < 0: none */
} oracle_config;

float oracle_powf(float x, float y);
double oracle_pow(double x, double y);
void oracle_powf_array(const float *x, float y, float *out, int64_t n);
void oracle_pow_array(const double *x, double y, double *out, int64_t n);
void oracle_rpowf_array(const float *x, double p, float *out, int64_t n);
void oracle_rpow_array(const double *x, double p, double *out, int64_t n);
const oracle_tableau *oracle_get_tableau(int method);

#define ORACLE_DECLARE(REAL, SFX)                                                                                      \
    void oracle_rhs_##SFX(const oracle_config *, const REAL *par, REAL t, const REAL *y, REAL *dy, int F);              \
    void oracle_erk_step_##SFX(const oracle_config *, const REAL *par, REAL t0, REAL dt, const REAL *y0,                \
                               const REAL *k0, REAL *k, REAL *y1, REAL *err, int F);                                    \
    void oracle_adapt_##SFX(const oracle_config *, REAL dt, const REAL *y0, const REAL *y1, const REAL *err, REAL prev, \
                            REAL prev_prev, REAL *out6, int F);                                                         \
    REAL oracle_initial_step_##SFX(const oracle_config *, const REAL *par, REAL t0, const REAL *y0, REAL t_end,         \
                                   REAL *f0, int F);                                                                    \
    void oracle_quartic_##SFX(const oracle_config *, REAL dt, const REAL *y0, const REAL *y1, const REAL *k, REAL *q,   \
                              int F);                                                                                   \
    void oracle_quartic_eval_##SFX(const REAL *q, REAL t0, REAL dt, REAL t, REAL *out, int F);                          \
    int oracle_solve_##SFX(const oracle_config *, int64_t B, int F, int E, const REAL *y0, const REAL *t_start,         \
                           const REAL *t_end, const REAL *t_eval, const REAL *dt0, const REAL *params, int P, REAL *ys, \
                           int64_t *n_steps, int64_t *n_accepted, int64_t *n_initialized, int64_t *status,              \
                           int64_t *n_f_evals, REAL *trace, int64_t trace_iters, int64_t trace_B,                      \
                           unsigned char *written /* [B,E] or NULL: 1 where the loop stored an evaluation point */);

ORACLE_DECLARE(float, f32)
ORACLE_DECLARE(double, f64)
#endif
