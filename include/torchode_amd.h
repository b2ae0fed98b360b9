/*
 * torchode_amd -- C ABI of the MI355X-native batch-parallel adaptive explicit
 * Runge-Kutta solve loop.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream and
 * allocates nothing.  All pointers are device pointers unless a comment says
 * otherwise; every array is contiguous (row-major) in the layout given.  An
 * entry point returns 0 on success and a negative TODE_E_* code otherwise;
 * tode_last_error() returns a human-readable message for the last failure on
 * the calling thread.  Work is enqueued on `stream` (a hipStream_t passed as
 * void*) and is asynchronous with respect to the host.
 *
 * "Reference" below is the torchode source tree (martenlienen/torchode 1.0.1);
 * each declaration names the Python interface it stands in for.
 */
#ifndef TORCHODE_AMD_H
#define TORCHODE_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TODE_ABI_VERSION 2

/* floating point type of data (y) and time (t) arrays */
enum { TODE_F32 = 0, TODE_F64 = 1 };
/* single step methods: reference single_step_methods/dopri5.py, tsit5.py */
enum { TODE_DOPRI5 = 0, TODE_TSIT5 = 1 };
/* step size controllers: reference step_size_controllers.py:260 (integral), :554 (PID) */
enum { TODE_CTRL_INTEGRAL = 0, TODE_CTRL_PID = 1 };
/* right-hand sides the persistent kernel evaluates itself */
enum { TODE_TERM_LINEAR_DECAY = 0, TODE_TERM_VAN_DER_POL = 1, TODE_TERM_LORENZ63 = 2 };
/* per-sample status codes: reference status_codes.py:9-13 */
enum {
    TODE_SUCCESS = 0,
    TODE_GENERAL_ERROR = 1,
    TODE_REACHED_DT_MIN = 2,
    TODE_REACHED_MAX_STEPS = 3,
    TODE_INFINITE_NORM = 4
};
/* Safety limit, not in the reference: a sample that reaches 2^22 steps stops with
 * TODE_GENERAL_ERROR (the reference's loop would never end; a kernel must). */
#define TODE_HARD_STEP_LIMIT (1 << 22)

/* return codes */
enum {
    TODE_OK = 0,
    TODE_E_INVALID = -1,     /* bad argument (null pointer, negative size, unknown enum) */
    TODE_E_UNSUPPORTED = -2, /* valid request outside what the kernels are built for */
    TODE_E_HIP = -3          /* a HIP runtime call failed */
};

/* Layout of the int32 flag block that tode_solve_builtin fills (device memory, 4 words). */
enum {
    TODE_FLAG_MAX_ITERATIONS = 0, /* max over samples of n_steps                        */
    TODE_FLAG_FIRST_FAILURE = 1,  /* first loop iteration with a non-success status, or */
                                  /* INT32_MAX                                          */
    TODE_FLAG_NON_MONOTONE = 2,   /* 1 if some sample's t_eval row is not monotone in   */
                                  /* its direction of time and no pending mask was given */
    TODE_FLAG_NEEDS_GENERAL = 3,  /* tode_solve_builtin_fast only: 1 if the batch needs the  */
                                  /* general entry point (see there)                     */
    TODE_FLAG_WORDS = 4
};

/*
 * Step size controller parameters.
 * Replaces the constructor arguments of IntegralController / PIDController
 * (reference step_size_controllers.py:263-287, 566-596).  atol and rtol are
 * rounded to float32 before use, as the reference stores them in float32
 * buffers.  The error norm is the RMS norm (reference :170-181).
 */
typedef struct tode_controller {
    int32_t kind; /* TODE_CTRL_* */
    int32_t has_dt_min;
    int32_t has_dt_max;
    int32_t reserved;
    double atol, rtol;
    double pcoeff, icoeff, dcoeff; /* PID only */
    double safety, factor_min, factor_max;
    double dt_min, dt_max;
} tode_controller;

/*
 * One whole solve of a batch of initial value problems with a built-in
 * right-hand side, in a single persistent kernel (one sample per lane).
 *
 * Replaces AutoDiffAdjoint.solve (reference adjoints.py:42-311) together with
 * everything it calls per iteration: ExplicitRungeKutta.step
 * (single_step_methods/runge_kutta.py:226-279), {Integral,PID}Controller.init /
 * adapt_step_size / merge_states (step_size_controllers.py:333-490, 678-835),
 * {Dopri5,Tsit5}.build_interpolation and FourthOrderPolynomialInterpolation.evaluate
 * (dopri5.py:53-60, tsit5.py:123-139, interpolation.py:138-175).
 *
 * Each sample runs until it reaches t_end, reports a non-success status, or has
 * taken `iteration_cap` steps.  The reference couples the samples of a batch in
 * two ways -- every sample is stepped until the slowest has finished, and the
 * first non-success status stops the whole batch -- which the caller restores
 * from the flag block: L = min(first_failure, max_iterations) is the iteration
 * at which the reference loop would have ended; if L < max_iterations the
 * caller runs the solve again with iteration_cap = L, then passes L to
 * tode_finalize_stats.
 */
typedef struct tode_solve_args {
    int32_t dtype;  /* TODE_F32 | TODE_F64, for data and time alike */
    int32_t method; /* TODE_DOPRI5 | TODE_TSIT5 */
    int32_t term;   /* TODE_TERM_* */
    int32_t n_features;        /* F */
    int32_t n_eval;            /* E; 0 means "report y(t_end) only" */
    int32_t n_params;          /* P: parameters per sample */
    int64_t batch;             /* B */
    int64_t max_steps;         /* < 0: unlimited (reference AutoDiffAdjoint max_steps) */
    int64_t iteration_cap;     /* < 0: unlimited */
    double term_scalars[4];    /* batch-uniform RHS constants (Lorenz: sigma, beta) */
    const void *y0;            /* [B,F] */
    const void *t_start;       /* [B], sample b at element b * t_start_stride */
    const void *t_end;         /* [B], sample b at element b * t_end_stride   */
    int64_t t_start_stride;    /* >= 1; 1 for a dense array, E for column 0 of t_eval */
    int64_t t_end_stride;      /* >= 1 */
    const void *t_eval;        /* [B,E] or NULL when E == 0 */
    const void *dt0;           /* [B] user initial step, or NULL to select one */
    const void *params;        /* [B,P] */
    void *ys;                  /* out [B,max(E,1),F] */
    void *y_idle;              /* out [B,F], used only when E == 0: value the reference
                                  reports for a sample that finished before iteration L */
    uint8_t *pending;          /* scratch [B,E] bytes, or NULL; needed only for t_eval rows
                                  that are not monotone in the direction of time */
    int32_t *n_steps;          /* out [B] */
    int32_t *n_accepted;       /* out [B] */
    int32_t *n_initialized;    /* out [B] */
    int32_t *status_last;      /* out [B] status at the sample's last own iteration */
    int32_t *status_idle;      /* out [B] status the sample reports in later iterations */
    int32_t *flags;            /* out [TODE_FLAG_WORDS] */
} tode_solve_args;

/* ABI version of the loaded library (== TODE_ABI_VERSION of the header it was built from). */
int tode_abi_version(void);

/* Message for the most recent non-zero return code on this host thread (host pointer). */
const char *tode_last_error(void);

/* See tode_solve_args. */
int tode_solve_builtin(const tode_solve_args *args, const tode_controller *controller, void *stream);

/*
 * Turns the per-sample outputs of tode_solve_builtin into what the reference
 * returns (adjoints.py:267-309): int64 stats and the final status of every
 * sample at loop iteration `last_iteration` (L above).  status[b] is
 * status_last[b] when n_steps[b] == L and status_idle[b] otherwise.  When
 * n_eval == 0, ys[b] is replaced by y_idle[b] for samples with n_steps[b] < L.
 */
int tode_finalize_stats(int64_t batch, int64_t last_iteration, const int32_t *n_steps, const int32_t *n_accepted,
                        const int32_t *n_initialized, const int32_t *status_last, const int32_t *status_idle,
                        int64_t *out_n_steps, int64_t *out_n_accepted, int64_t *out_n_initialized, int64_t *out_status,
                        int32_t dtype, int32_t n_features, int32_t n_eval, void *ys, const void *y_idle, void *stream);

/*
 * The same solve as tode_solve_builtin for the common case, in one kernel launch
 * with no finalisation step: evaluation points given (n_eval > 0), no dt_min /
 * dt_max, and a batch in which every sample succeeds.  Uses of `args`: all
 * inputs, `ys` and `flags`; the int32 per-sample outputs, `y_idle`, `pending`
 * and `iteration_cap` are ignored.  The reference's int64 stats and status are
 * written directly (adjoints.py:267-294).
 *
 * On return (after stream synchronisation) flags[TODE_FLAG_MAX_ITERATIONS] is
 * the loop's iteration count, and flags[TODE_FLAG_NEEDS_GENERAL] == 1 means the
 * batch left the common case (a non-success status, max_steps reached, a t_eval
 * row that is not monotone in its direction of time, or a sample that ended
 * past t_end); every output is then unspecified and the caller must repeat the
 * solve with tode_solve_builtin.  Results are bit-identical to
 * tode_solve_builtin + tode_finalize_stats whenever the flag stays 0.
 * Returns TODE_E_UNSUPPORTED for n_eval == 0, dt_min / dt_max, or n_eval too
 * large for on-chip staging.
 */
int tode_solve_builtin_fast(const tode_solve_args *args, const tode_controller *controller, int64_t *out_n_steps,
                            int64_t *out_n_accepted, int64_t *out_n_initialized, int64_t *out_status, void *stream);

/* ------------------------------------------------------------------------- */
/* Per-step kernels around a right-hand side that lives outside the library   */
/* ------------------------------------------------------------------------- */

/* Layout of the int32 flag block of a stepwise solve (device memory). */
enum {
    TODE_STEP_FLAG_STOPPED = 0,     /* 1 once the loop has ended on the device               */
    TODE_STEP_FLAG_ITERATIONS = 1,  /* loop iterations completed before it ended             */
    TODE_STEP_FLAG_ANY_RUNNING = 2, /* scratch of the current iteration                      */
    TODE_STEP_FLAG_ANY_FAILURE = 3, /* 1 once any sample reported a non-success status       */
    TODE_STEP_FLAG_WORDS = 4
};

/*
 * Device-resident state of one solve whose right-hand side f is evaluated by
 * the caller (any framework) between kernels.  The caller owns every buffer
 * for the duration of the solve.  Data and time share one dtype.
 *
 * Replaces the locals of AutoDiffAdjoint.solve (reference adjoints.py:59-126),
 * ERKState / ERKInterpolationData (single_step_methods/runge_kutta.py:161-172)
 * and PIDState (step_size_controllers.py:493-551).
 *
 * Protocol of one solve on one stream (no host synchronisation required
 * between calls):
 *   k[0] <- f(t_start, y0)
 *   tode_step_begin(phase 0)            with dt0 == NULL: ystage[1], tnode <- start-step probe
 *   [ k[1] <- f(tnode, ystage[1]);  tode_step_begin(phase 1) ]      only when dt0 == NULL
 *   repeat:  for s = 1..6:  tode_step_stage(s);  k[s] <- f(tnode, ystage[s])
 *            tode_step_finish()
 *   The caller reads `flags` whenever it likes; after TODE_STEP_FLAG_STOPPED is
 *   set, further stage/finish calls are no-ops.  tode_step_stats converts the
 *   counters.  k[0] must point at k0 from the first stage call on (begin
 *   copies f(t_start, y0) there).
 */
typedef struct tode_step_state {
    int32_t dtype;      /* TODE_F32 | TODE_F64 */
    int32_t method;     /* TODE_DOPRI5 | TODE_TSIT5 */
    int32_t n_features; /* F */
    int32_t n_eval;     /* E; 0: report y(t_end) only */
    int64_t batch;      /* B */
    int64_t max_steps;  /* < 0: unlimited */
    const void *y0;      /* [B,F] */
    const void *t_start; /* [B] */
    const void *t_end;   /* [B] */
    const void *t_eval;  /* [B,E] or NULL */
    void *t;             /* [B]   current time            */
    void *dt;            /* [B]   current step            */
    void *y;             /* [B,F] current state           */
    void *k0;            /* [B,F] FSAL derivative f(t, y) */
    void *ratio_prev;    /* [B] last accepted error ratio (PID history, data dtype) */
    void *ratio_pprev;   /* [B] ... and the one before                             */
    int32_t *running;    /* [B] */
    int32_t *cursor;     /* [B] index of the first evaluation point still pending  */
    int32_t *n_steps;    /* [B] */
    int32_t *n_accepted; /* [B] */
    int32_t *status;     /* [B] status of the latest iteration */
    int32_t *monotone;   /* [B] 1 if the sample's t_eval row is monotone in its direction */
    uint8_t *pending;    /* [B,E] 1 while an evaluation point has not been written */
    void *ys;            /* out [B,max(E,1),F] */
    int32_t *flags;      /* [TODE_STEP_FLAG_WORDS] */
    void *ystage[7];     /* [B,F] each: input of stage s (index 0 unused); ystage[6] is y1 */
    const void *k[7];    /* [B,F] each: f at stage s, written by the caller; k[0] == k0   */
    void *tnode;         /* [B] time of the stage that was just prepared */
} tode_step_state;

/*
 * Start of a stepwise solve.  phase 0 resets the flag block and, with a user
 * step dt0 ([B], may be NULL), initialises the loop state from k[0]; without
 * dt0 it prepares the second evaluation of the start-step selection
 * (reference step_size_controllers.py:431-490, 776-835).  phase 1 (only when
 * dt0 == NULL) finishes the selection from k[1] and initialises the loop state
 * (adjoints.py:59-126).
 */
int tode_step_begin(const tode_step_state *state, const tode_controller *controller, const void *dt0, int phase, void *stream);

/*
 * Stage `stage` (1..6): ystage[stage] = fma(dt, sum_j a[stage][j] k[j], y) and
 * tnode = fma(c[stage], dt, t).  Replaces the body of the stage loop of
 * ExplicitRungeKutta.step (reference single_step_methods/runge_kutta.py:259-262).
 */
int tode_step_stage(const tode_step_state *state, const tode_controller *controller, int stage, void *stream);

/*
 * Everything after the sixth stage of one loop iteration, fused into one pass
 * per sample: error estimate (runge_kutta.py:265-272), error ratio, accept /
 * reject, PI/PID proposal, dt_min / dt_max and status
 * (step_size_controllers.py:370-429, 715-774), counters, dense output at the
 * evaluation points the step passed (adjoints.py:215-234 with
 * tsit5.py:123-139 / dopri5.py:53-60 / interpolation.py:25-40), state and FSAL
 * update, running flag, dt clamp and controller history (adjoints.py:150-255),
 * followed by the loop-continuation decision (adjoints.py:186-190).
 */
int tode_step_finish(const tode_step_state *state, const tode_controller *controller, void *stream);

/* int32 counters of a stepwise solve -> the int64 stats and status the reference returns
 * (adjoints.py:267-292). */
int tode_step_stats(const tode_step_state *state, int64_t *out_n_steps, int64_t *out_n_accepted, int64_t *out_n_initialized,
                    int64_t *out_status, void *stream);

/*
 * Which kernel tode_solve_builtin_fast launches (per host thread); no counterpart in the
 * reference.  0 (default): two wavefronts per 64 samples (a stepper and a dense-output
 * evaluator) while the batch would otherwise leave SIMDs with at most two wavefronts, one
 * wavefront per 64 samples above that; 1: always one wavefront; 2: two wavefronts or
 * TODE_E_UNSUPPORTED.  All variants produce identical bits.
 */
int tode_set_fast_kernel_variant(int variant);

/*
 * Kernel timing for benchmarks and profiling; no counterpart in the reference.
 * While enabled (per host thread), tode_solve_builtin and tode_solve_builtin_fast record a HIP event on
 * `stream` directly before and directly after its solve kernel.
 * tode_last_solve_kernel_ms waits for the second event of the most recent
 * launch made by the calling thread and writes the elapsed milliseconds of
 * that one kernel; it returns TODE_E_INVALID if timing was off or nothing was
 * launched.
 */
int tode_set_kernel_timing(int enable);
int tode_last_solve_kernel_ms(float *out_ms);
/* Name of the solve kernel most recently launched by the calling thread ("" if none), e.g.
 * "tode::solve_pair_kernel"; the same for every template instance of a kernel. */
const char *tode_last_solve_kernel_name(void);

#ifdef __cplusplus
}
#endif
#endif /* TORCHODE_AMD_H */
