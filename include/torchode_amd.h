/*
 * torchode_amd -- C ABI of the MI355X-native batch-parallel adaptive explicit
 * Runge-Kutta solve loop.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream.  None
 * allocates per call; tode_solve_builtin_fast_sync allocates its flag words once
 * per device on its first call there (see its comment), the others never.  All
 * pointers are device pointers unless a comment says
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

#define TODE_ABI_VERSION 23

/* floating point type of data (y) and time (t) arrays */
enum { TODE_F32 = 0, TODE_F64 = 1 };
/* A dtype argument when time and data differ (reference problems.py:44-56, tests/dtype_stability_test.py):
 * TODE_DTYPES(data, time); a plain TODE_F32 / TODE_F64 means both.  Time: t, dt, t_start, t_end, t_eval, a user's
 * dt0 and everything derived (node times, next step size, step limits).  Data: y, parameters of the term,
 * derivatives, coefficients, error norms and ratios, ys. */
#define TODE_DTYPE_PAIR 0x100
#define TODE_DTYPES(data, time) (TODE_DTYPE_PAIR | (data) | ((time) << 4))
/* single step methods: reference single_step_methods/dopri5.py, tsit5.py, heun.py, euler.py */
enum { TODE_DOPRI5 = 0, TODE_TSIT5 = 1, TODE_HEUN = 2, TODE_EULER = 3 /* the last two: per-step entry points only */ };
/* step size controllers: reference step_size_controllers.py:260 (integral), :554 (PID) */
enum { TODE_CTRL_INTEGRAL = 0, TODE_CTRL_PID = 1, TODE_CTRL_FIXED = 2 /* per-step entry points only */ };
/* right-hand sides the persistent kernel evaluates itself */
enum {
    TODE_TERM_LINEAR_DECAY = 0,       /* dy/dt = -k y, k [B,F] */
    TODE_TERM_VAN_DER_POL = 1,        /* F = 2, mu [B] */
    TODE_TERM_LORENZ63 = 2,           /* F = 3, rho [B]; sigma, beta in term_scalars */
    TODE_TERM_REACTION_DIFFUSION = 3, /* F = N*N periodic grid (N = 16, 32 or 64; float32 also 128), du/dt = D lap(u) + u (1 - u),
                                         D [B]; float32 or float64 (time and data alike), tode_solve_builtin_fast only */
    TODE_TERM_MLP = 4                 /* F = 1 ... 64: tanh([y, t] W1^T + b1) W2^T + b2 with up to 256 hidden units,
                                         weights in shared_params as packed by tode_mlp_pack_weights[_for]; float32,
                                         tode_solve_builtin_fast only */
};
/* what the matrix cores take as inputs in the MLP kernel; accumulation, biases, tanh and the solver are float32 */
enum { TODE_MLP_INPUTS_F32 = 0, TODE_MLP_INPUTS_BF16 = 1 };
/* number of 32-bit words tode_mlp_pack_weights writes for either */
#define TODE_MLP_PACKED_SIZE (152 * 256)
#define TODE_MLP_PACKED_SIZE_BF16 (92 * 256)
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
/*
 * Optional record of the loop state, written by tode_solve_builtin (the general kernel) and, for the three small
 * systems with evaluation points, by tode_solve_builtin_fast and its _sync / _static forms (the two-wavefront or the
 * single-wavefront kernel: the solve and its record in one launch) when tode_solve_args.record points to one: entry i
 * holds what the reference's loop variables hold before iteration i
 * (adjoints.py:135-260: t, dt, y, the first-same-as-last derivative, the PID controller's two previous error
 * ratios, `running`, `n_accepted`), entry n_steps[b] the sample's final state, and the entries after it that final
 * state again with running = 0 -- a finished sample keeps its state while the batch goes on.  It is what a reverse
 * sweep over the iterations starts from (tode_step_finish_backward / tode_step_stage_backward), the counterpart of the
 * operation graph that torch.autograd keeps for the reference's loop.  All arrays are device memory with
 * `capacity` entries of the batch each, entry-major: t, dt [capacity, B] in the time type; y, k0 [capacity, B, F] and
 * prev, pprev [capacity, B] in the data type; running, n_accepted [capacity, B] int32.  capacity must be at least
 * 1 + the iterations the solve takes (args->iteration_cap + 1 when a cap is set, which is how a caller that has
 * solved the problem once sizes it); a sample whose steps do not fit stops recording and raises
 * TODE_FLAG_NEEDS_GENERAL in the flag block.  A caller without that count gives the fast entry point a record sized
 * from a similar solve and repeats the solve if the flag comes back (TODE_FLAG_MAX_ITERATIONS then says what fits).
 */
typedef struct tode_solve_record {
    int64_t capacity;
    void *t, *dt, *y, *k0, *prev, *pprev;
    int32_t *running, *n_accepted;
} tode_solve_record;

typedef struct tode_solve_args {
    int32_t dtype;  /* TODE_F32 | TODE_F64 for data and time alike; TODE_DTYPES(data, time) where they differ:
                       tode_solve_builtin and tode_solve_builtin_auto take it for the three small systems (the
                       general kernel is built for all four pairs), the fast entry points return TODE_E_UNSUPPORTED */
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
    const void *shared_params; /* [n_shared_params] right-hand side parameters shared by the batch, or NULL */
    int64_t n_shared_params;   /* TODE_TERM_MLP: TODE_MLP_PACKED_SIZE[_BF16], the words tode_mlp_pack_weights wrote */
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
    const tode_solve_record *record; /* NULL, or where tode_solve_builtin / tode_solve_builtin_fast keep the loop state
                                        of every iteration (HOST pointer to the struct; tode_solve_builtin_auto
                                        ignores it) */
} tode_solve_args;

/* ABI version of the loaded library (== TODE_ABI_VERSION of the header it was built from). */
int tode_abi_version(void);

/* sha256 (hex, host pointer) of the sources and compiler flags the loaded library was built from, as the build
 * script computes it; empty for a build that did not pass one.  A loader compares it with the sources it finds
 * beside the library, so that an edited kernel is never tested through a stale binary. */
const char *tode_source_hash(void);

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
 * with no finalisation step: evaluation points given (n_eval > 0; for
 * n_eval == 0 see below), no dt_min / dt_max, and a batch in which every sample
 * succeeds.  Uses of `args`: all inputs, `ys` and `flags` (and `y_idle` when
 * n_eval == 0); the int32 per-sample outputs, `pending` and `iteration_cap` are
 * ignored.  The reference's int64 stats and status are written directly
 * (adjoints.py:267-294).
 *
 * On return (after stream synchronisation) flags[TODE_FLAG_MAX_ITERATIONS] is
 * the loop's iteration count, and flags[TODE_FLAG_NEEDS_GENERAL] == 1 means the
 * batch left the common case (a non-success status, max_steps reached, a t_eval
 * row that is not monotone in its direction of time, a sample that ended on a
 * non-finite state or, with n_eval == 0, past t_end); every output is then
 * unspecified and the caller must repeat the solve with tode_solve_builtin.
 * (With evaluation points a sample that lands past t_end, t + (t_end - t)
 * rounded upwards, stays in the kernel: the reference steps it once more with
 * the step t_end - t, which shows in that step's status alone, and the kernel
 * computes that step and looks at its error ratio.)  Results are bit-identical to
 * tode_solve_builtin + tode_finalize_stats whenever the flag stays 0.
 * Returns TODE_E_UNSUPPORTED for dt_min / dt_max, or n_eval too large for
 * on-chip staging.
 *
 * n_eval == 0 (the reference's t_eval=None, adjoints.py:296-311: the end point
 * alone, ys of shape [B,1,F]) is covered for the small systems (linear decay,
 * Van der Pol, Lorenz) in batches of up to TODE_END_ONLY_MAX_BATCH samples and
 * for the grid and MLP terms; otherwise TODE_E_UNSUPPORTED.  `t_eval` may then be null and `y_idle` [B,F]
 * must be given: the kernel leaves in ys[b] the dense output of sample b's last
 * step at t_end and in y_idle[b] its final state, and the caller, once it has
 * read the flags, finishes with tode_select_end_point(...,
 * flags[TODE_FLAG_MAX_ITERATIONS], ...).
 */
#define TODE_END_ONLY_MAX_BATCH (2048 * 64)
int tode_solve_builtin_fast(const tode_solve_args *args, const tode_controller *controller, int64_t *out_n_steps,
                            int64_t *out_n_accepted, int64_t *out_n_initialized, int64_t *out_status, void *stream);

/*
 * tode_solve_builtin_fast for a caller that needs the flag block on the host at
 * once, as the reference's loop does (its stats["n_f_evals"] is a CPU tensor,
 * terms.py:41-63, and adjoints.py:197-201 synchronises on the loop's state):
 * the same kernels, but `args->flags` is not used (may be null).  The kernel
 * works on flag words the library owns (allocated once per device, on the
 * first call), its last workgroup stores them into pinned host memory, and
 * this call returns when they have arrived there, with the TODE_FLAG_WORDS
 * values in the host array `flags_out`.  That saves the launch that resets the
 * flag block and the device-to-host copy.  Only the flag words are on the host
 * when the call returns: ys and the four stat arrays are complete in stream
 * order, as for tode_solve_builtin_fast (work enqueued on `stream` afterwards,
 * or a stream synchronisation, sees them; the returned call by itself does not
 * make other workgroups' stores visible to the host or to other streams).  Safe to
 * call from several host threads and on several streams at once.  With
 * n_eval == 0 this call also enqueues tode_select_end_point.  Where
 * tode_solve_builtin_fast would refuse a small system for its shape (n_eval
 * == 0 or n_eval too large, in a batch that the two-wavefront kernel does not
 * take), this call launches no kernel and reports
 * flags_out[TODE_FLAG_NEEDS_GENERAL] = 1.
 */
int tode_solve_builtin_fast_sync(const tode_solve_args *args, const tode_controller *controller, int64_t *out_n_steps,
                                 int64_t *out_n_accepted, int64_t *out_n_initialized, int64_t *out_status, void *stream,
                                 int32_t *flags_out);

/*
 * tode_solve_builtin_fast for a caller that cannot allocate.  No counterpart in
 * the reference; it is for code under HIP graph capture, tight serving loops
 * and harnesses that forbid allocation calls: this call performs no hipMalloc /
 * hipFree / hipHostMalloc and no allocating library routine, now or on its first
 * use.  The device memory the solve needs beyond its inputs and outputs -- the
 * working flag words with the count of finished workgroups, and, when n_eval ==
 * 0, the [B,F] staging area of the final states -- lies in a static device array
 * of the library (256 + TODE_STATIC_STAGING_BYTES bytes, one copy per GPU the
 * library runs on, held until the process ends).  `args->flags` and
 * `args->y_idle` are not used (may be null).  The kernels are those of
 * tode_solve_builtin_fast and the results are bit-identical to it; the flag
 * block is written to `flags_out` (DEVICE memory, TODE_FLAG_WORDS int32) and is
 * valid in stream order, like ys and the stats; the caller reads it when it
 * likes (flags_out[TODE_FLAG_NEEDS_GENERAL] as for tode_solve_builtin_fast).
 * With n_eval == 0 the call also enqueues the end point selection
 * (tode_select_end_point), which reads the iteration count from flags_out on
 * the device, so ys is final without a host round trip.
 *
 * Limit: with n_eval == 0, B * F * sizeof(value) must not exceed
 * TODE_STATIC_STAGING_BYTES; beyond that the call returns TODE_E_UNSUPPORTED
 * and launches nothing.  With n_eval > 0 the array sets no limit.  Shapes that
 * tode_solve_builtin_fast refuses are refused here with the same code.
 *
 * Every call on a GPU uses that GPU's one array, so calls must not overlap on a
 * GPU.  Calls in a row on one stream need nothing: the stream orders them, and
 * each call resets the words it uses by a kernel in front of the solve kernel.
 * Host threads take turns inside the call.  A call on another stream than the
 * GPU's last call is refused with TODE_E_UNSUPPORTED, and launches nothing,
 * while that last call's work has not finished (an event recorded behind every
 * call is looked at, no waiting); the caller synchronises and calls again.
 * Under stream capture nothing runs at the time of the call, so nothing is
 * checked: whoever replays the graph keeps the replays apart from other calls
 * on that GPU.  The array's address is looked up and the event made on the
 * first call on a device (hipGetSymbolAddress and hipEventCreate: no device
 * memory is allocated); a caller that captures a graph makes one call before
 * capturing.
 */
#define TODE_STATIC_STAGING_BYTES (2 << 20)
int tode_solve_builtin_fast_static(const tode_solve_args *args, const tode_controller *controller, int64_t *out_n_steps,
                                   int64_t *out_n_accepted, int64_t *out_n_initialized, int64_t *out_status,
                                   int32_t *flags_out, void *stream);

/*
 * The whole of AutoDiffAdjoint.solve (reference adjoints.py:42-311) for a
 * built-in term in one call: the one-kernel path where the problem is in its
 * shape (tode_solve_builtin_fast_sync), else or after it reported
 * TODE_FLAG_NEEDS_GENERAL the general kernel (tode_solve_builtin, launched
 * again with a pending mask for rows of evaluation points that are not
 * monotone, and again with an iteration cap when some sample reported a
 * non-success status, adjoints.py:229-238), then tode_finalize_stats.  On
 * return ys and the four int64 [B] outputs hold what the reference returns and
 * *iterations (HOST memory) the number of loop iterations L, from which the
 * caller forms stats["n_f_evals"] = (dt0 given ? 1 : 2) + 6 L (terms.py:41-63).
 *
 * The call synchronises with the stream (once in the common case), as the
 * reference's loop does in every iteration.  It allocates nothing: flag words,
 * int32 counters, the pending mask and the idle end points live in `workspace`,
 * DEVICE memory of at least tode_solve_workspace_bytes(args) bytes that the
 * caller provides and may reuse for the next call on the same stream.
 * args->flags, pending, y_idle, the five int32 outputs and iteration_cap are
 * not read.  allow_one_kernel = 0 sends the three small systems to the
 * general kernel directly (same results).
 *
 * Returns TODE_E_UNSUPPORTED, with nothing written that the caller may rely
 * on, where no whole-solve kernel covers the problem (reaction-diffusion and
 * MLP outside the shapes named at TODE_TERM_*, or a batch of theirs with a
 * non-success status, non-monotone rows or step size limits): the caller runs
 * the loop through the per-step or the operator entry points instead.
 */
int64_t tode_solve_workspace_bytes(const tode_solve_args *args);
int tode_solve_builtin_auto(const tode_solve_args *args, const tode_controller *controller, int64_t *out_n_steps,
                            int64_t *out_n_accepted, int64_t *out_n_initialized, int64_t *out_status, void *workspace,
                            int64_t workspace_bytes, int32_t allow_one_kernel, void *stream, int64_t *iterations);

/*
 * Last step of a solve without evaluation points through tode_solve_builtin_fast
 * (adjoints.py:296-311): the reference evaluates the interpolant of the batch's
 * LAST iteration at t_end, and a sample that had finished earlier took a
 * zero-length step in that iteration, whose interpolant is its final state.
 * ys[b] = y_idle[b] for every sample with n_steps[b] < last_iteration; the
 * others keep the dense output of their last step.
 */
int tode_select_end_point(int64_t batch, int32_t n_features, int32_t dtype, int64_t last_iteration, const int64_t *n_steps, void *ys,
                          const void *y_idle, void *stream);

/*
 * Weights of TODE_TERM_MLP in the order the solve kernel loads them into
 * registers (each thread of a workgroup reads its own values, contiguous across
 * a wavefront).  `raw`: W1 [H x 65] | b1 [H] | W2 [64 x H] | b2 [64] for a
 * network of H hidden units, 1 <= H <= 256, row-major float32 on the device,
 * n_raw = 130 H + 64 (33344 for H = 256) -- the parameters of the user's `f` as
 * a torch module holds them (terms.py:13-19 takes any callable).  The kernel
 * always works on 256 units: those from H on are packed with zero weights and
 * a zero bias and add exact zeros to every sum.
 * `packed`: TODE_MLP_PACKED_SIZE (matrix_inputs = TODE_MLP_INPUTS_F32) or
 * TODE_MLP_PACKED_SIZE_BF16 (TODE_MLP_INPUTS_BF16: W1 and W2 rounded to
 * bfloat16, two per word) 32-bit words on the device; pass it as shared_params
 * with that count as n_shared_params, which also selects the kernel.  With
 * bfloat16 inputs the solve is a reduced-precision variant of its own (the
 * stage inputs and hidden activations are rounded as well): results differ
 * from the float32 path at the 1e-3 level.  Pack once per change of the
 * weights, not per solve.
 */
int tode_mlp_pack_weights(const void *raw, int64_t n_raw, int32_t matrix_inputs, void *packed, void *stream);

/*
 * The same for a network on n_features = 1 ... 64 state values (the solve
 * then takes n_features of that size and rows of that many values in y0 and
 * ys): `raw` is W1 [H x (n_features + 1)] | b1 [H] | W2 [n_features x H] |
 * b2 [n_features], n_raw = (2 n_features + 2) H + n_features.  The kernel always
 * works on 64 values per sample: the state values from n_features on are zero,
 * their weights are packed as zeros, and the root mean squares divide by
 * n_features, so the sums hold only exact zeros beyond the network's own terms.
 * `packed` has the same size as for 64 features.  (Rows of a multiple of four values
 * are loaded and stored 16 bytes at a time, others value by value.)
 * tode_mlp_pack_weights(...) == tode_mlp_pack_weights_for(..., 64, ...).
 */
int tode_mlp_pack_weights_for(const void *raw, int64_t n_raw, int32_t n_features, int32_t matrix_inputs, void *packed, void *stream);

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
 * for the duration of the solve.  Data and time may have different dtypes
 * (`dtype` and `time_dtype` below).
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
 *   Heun and Euler keep no derivative from one step to the next (heun.py, euler.py): every iteration starts with
 *   k[0] <- f(t, y) of the current state, then stage 1 (Heun only), then tode_step_finish; ystage[6] is scratch
 *   for the step's result (rows of fewer than 64 features; longer rows need none).
 *   The caller reads `flags` (a synchronisation) or `host_flags` (none) whenever it
 *   likes; after TODE_STEP_FLAG_STOPPED is set, further stage/finish calls are no-ops.  tode_step_stats converts the
 *   counters.  k[0] must point at k0 from the first stage call on (begin
 *   copies f(t_start, y0) there).
 */
typedef struct tode_step_state {
    int32_t dtype;      /* TODE_F32 | TODE_F64: y0, y, k0, ratio_prev/pprev, ys, ystage, k */
    int32_t time_dtype; /* TODE_F32 | TODE_F64: t_start, t_end, t_eval, t, dt, tnode and a user dt0
                           (problems.py:44-56: time and data may differ) */
    int32_t method;     /* TODE_DOPRI5 | TODE_TSIT5 | TODE_HEUN | TODE_EULER */
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
    int32_t *host_flags; /* NULL, or two int32 in pinned host memory that the device can write: every
                            tode_step_finish leaves there TODE_STEP_FLAG_STOPPED and
                            TODE_STEP_FLAG_ITERATIONS as of its iteration, so that the host can see the loop
                            end by reading its own memory, without a synchronisation */
    const void *fixed_dt; /* [B] time dtype, TODE_CTRL_FIXED only: the step every running sample takes
                             (step_size_controllers.py:116-167: every step is accepted and the next step
                             is dt0 again, whatever the last one was clamped to) */
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
 * Which of its two kernels for the small systems tode_solve_builtin_fast launches (per host thread); no counterpart
 * in the reference.  A hook for tests and profiles, which have to address each kernel on inputs of their choice.
 * 0 (default): two wavefronts per 64 samples (a stepper and a dense-output evaluator) while the batch would
 * otherwise leave SIMDs with at most two wavefronts, one wavefront per 64 samples above that; 1: always one
 * wavefront; 2: two wavefronts or TODE_E_UNSUPPORTED.  Both kernels produce identical bits.
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

/* ------------------------------------------------------------------------------------------
 * Reverse of one loop iteration of the per-step kernels (gradients through the loop)
 * ------------------------------------------------------------------------------------------
 * Replaces what autograd does for the reference when AutoDiffAdjoint.solve runs under grad mode
 * (reference adjoints.py:33-40, 111-113, 145-147: the loop is torch operations, recorded as they
 * run).  The caller keeps the loop state of every iteration during the forward solve, walks the
 * iterations in reverse and, for each, recomputes the stage values with tode_step_stage and its
 * own f, then calls
 *   tode_step_finish_backward        cotangents of the state after the iteration and of the
 *                                    evaluation points it wrote  ->  g_k[0..6], g_y, g_y1, g_t,
 *                                    g_dt, g_prev, g_pprev (overwritten) and the time gradients
 *                                    (accumulated)
 *   for s = 6 .. 1:
 *       (g_ystage, g_tnode, ...) = vector-Jacobian product of the caller's f at stage s with g_k[s]
 *       (for s = 6, g_ystage += g_y1)
 *       tode_step_stage_backward(s)  adds to g_y, g_k[j < s], g_t, g_dt
 * after which (g_y, g_k[0], g_t, g_dt, g_prev, g_pprev) are the cotangents of the state before the
 * iteration.  Rows of fewer than 64 features: one thread per sample; longer rows: one wavefront per sample.
 */
typedef struct tode_step_adjoint {
    int32_t dtype;           /* TODE_F32 | TODE_F64: data (y, k, history, their cotangents, grad_ys) */
    int32_t time_dtype;      /* TODE_F32 | TODE_F64: times and steps and their cotangents */
    int32_t method;          /* TODE_DOPRI5 | TODE_TSIT5 */
    int32_t n_features;      /* F */
    int32_t n_eval;          /* E; 0: the end point alone */
    int32_t iteration;       /* index of this loop iteration */
    int32_t through_control; /* 1: the proposed step is a function of the inputs (AutoDiffAdjoint's
                                backprop_through_step_size_control, adjoints.py:111-113); 0: a constant */
    int32_t end_point;       /* n_eval == 0 only: 1 in the loop's last iteration, whose interpolant gives ys */
    int64_t batch;           /* B */
    /* the problem and the forward values of the iteration */
    const void *t_start, *t_end; /* [B] */
    const void *t_eval;          /* [B,E] or NULL */
    const void *t, *dt;          /* [B] state before the iteration */
    const void *y;               /* [B,F] */
    const void *ratio_prev, *ratio_pprev; /* [B] */
    const int32_t *running;      /* [B] before the iteration (unused by the kernels, kept for callers' checks; may be NULL) */
    const int32_t *moved;        /* [B] 1 where the step was accepted for a running sample */
    const int32_t *running_next; /* [B] running after the iteration */
    const void *k[7];            /* [B,F] each; k[0] is the state's FSAL derivative */
    const void *y1;              /* [B,F] input of the last stage = the step's result */
    const void *fixed_dt;        /* [B] TODE_CTRL_FIXED only */
    const int32_t *hit_iteration;/* [B,E] iteration that wrote each evaluation point, -1 for none; NULL when E == 0 */
    const void *grad_ys;         /* [B,max(E,1),F] cotangent of the solve's ys */
    /* cotangents of the state after the iteration; NULL stands for zeros */
    const void *a_t, *a_dt;      /* [B] */
    const void *a_y, *a_k0;      /* [B,F] */
    const void *a_prev, *a_pprev;/* [B] */
    /* results, overwritten by tode_step_finish_backward and added to by tode_step_stage_backward */
    void *g_k[7];                /* [B,F] each */
    void *g_y, *g_y1;            /* [B,F] */
    void *g_t, *g_dt;            /* [B] */
    void *g_prev, *g_pprev;      /* [B] */
    /* gradients of the problem's times, added to; NULL: not wanted */
    void *g_t_start, *g_t_end;   /* [B] */
    void *g_t_eval;              /* [B,E] */
    void *g_fixed_dt;            /* [B] */
} tode_step_adjoint;

int tode_step_finish_backward(const tode_step_adjoint *adjoint, const tode_controller *controller, void *stream);
int tode_step_stage_backward(const tode_step_adjoint *adjoint, const tode_controller *controller, int stage, const void *g_ystage,
                             const void *g_tnode, void *stream);

/*
 * The reverse sweep over a whole recorded solve with one of the three small built-in systems, in one kernel (one
 * thread per sample walks its iterations from the last to the first).  It stands for the backward pass that
 * torch.autograd runs over the reference's loop (adjoints.py:33-40, 111-113, 135-260), and for the sequence
 * tode_step_stage / f / tode_step_finish_backward / f's vector-Jacobian product / tode_step_stage_backward per
 * iteration above, with the right-hand side and its vector-Jacobian product evaluated in the kernel.
 *
 * args: the forward problem as for tode_solve_builtin (y0 is not read; t_start / t_end with their strides; dtype one of TODE_F32 /
 * TODE_F64; method Dopri5 or Tsit5; controller integral or PID), with args->record pointing to the record the forward
 * pass wrote.  All pointers below are device memory.  Nothing is allocated; the call only enqueues.
 */
typedef struct tode_solve_adjoint {
    const void *grad_ys;           /* [B, max(E,1), F] cotangent of ys */
    const int32_t *points_by_iteration; /* [B,E]: each sample's evaluation points ordered by the iteration that wrote them */
    const int32_t *iterations_sorted;   /* [B,E]: those iterations in the same order, ascending; -1 (first) for a point that
                                           no iteration wrote.  Both NULL when E == 0 -- or to have the library work
                                           them out from the record's times (a kernel of its own in front of the sweep,
                                           into `scratch`) */
    int64_t iterations;            /* L: iterations of the loop; the record's entries 0..L are read */
    int32_t through_control;       /* as in tode_step_adjoint */
    int32_t through_start;         /* 0: the results are the cotangents of the loop's first state.  1: the kernel also
                                      carries them through the start of the loop (y = y0, the first derivative
                                      f(t_start, y0), and -- with through_control and args->dt0 == NULL -- the first
                                      step from the start rule, step_size_controllers.py:431-490 / 776-835, clamped to
                                      the time range): a_y is then the cotangent of y0 and g_params includes the
                                      start's share.  The times count as constants in that part, so a caller that
                                      wants g_t_start / g_t_end passes 0 and does the start itself.  args->dt0 is not
                                      read, only looked at: non-NULL says that the first step was the caller's */
    void *scratch;                 /* tode_solve_backward_scratch_bytes(args) bytes (two int32 lists of [B,E]); looked at
                                      only when the two lists above are NULL and E > 0 */
    int64_t scratch_bytes;
    /* results: cotangents of the loop state before the first iteration (y, the first-same-as-last derivative
       f(t_start, y0), t, the first step, the controller's history) ... */
    void *a_y, *a_k0;              /* [B,F] */
    void *a_t, *a_dt, *a_prev, *a_pprev; /* [B] */
    void *g_params;                /* ... and of the term's per-sample parameters [B,P] */
    void *g_t_start, *g_t_end;     /* [B], added to; NULL: not wanted */
    void *g_t_eval;                /* [B,E], added to; NULL: not wanted */
} tode_solve_adjoint;
int64_t tode_solve_backward_scratch_bytes(const tode_solve_args *args);
int tode_solve_builtin_backward(const tode_solve_args *args, const tode_controller *controller, const tode_solve_adjoint *adjoint, void *stream);

/* ------------------------------------------------------------------------------------------
 * Protocol operators.
 *
 * The reference's solve loop is written against plug-in protocols (SingleStepMethod,
 * StepSizeController, LocalInterpolation; reference single_step_methods/base.py:20-89,
 * step_size_controllers.py:16-113, interpolation.py:43-45), and users may supply their own
 * implementation of any of them.  The operators below are what the package's own
 * implementations of those protocol methods call, one kernel each, so that any mix of
 * library and user-supplied parts runs through the same loop.  Time and data may have different
 * floating point types (reference problems.py:44-56, tests/dtype_stability_test.py), see TODE_DTYPES.
 * All pointers are device pointers except the `const double *` coefficient arrays, which are
 * host arrays read before the call returns.  Arrays are dense row-major.
 * ------------------------------------------------------------------------------------------ */
#define TODE_MAX_STAGES 16
/* dtype argument of the operators: TODE_F32, TODE_F64 or TODE_DTYPES(data, time), defined at the top of this file. */
enum { TODE_NORM_RMS = 0, TODE_NORM_MAX = 1 }; /* reference step_size_controllers.py:170-186 */

/* Coefficients the kernels use for Dopri5 / Tsit5 (reference dopri5.py:11-44, tsit5.py:11-114), as doubles:
 * c [7], a [7*7] row-major (strictly lower triangle; row 6 is b), b_err [7], b_other [3*7] with *n_other rows set
 * (Dopri5: the mid-point weights; Tsit5: the theta^2..theta^4 dense output weights).  Host arrays. */
int tode_tableau(int32_t method, double *c, double *a, double *b_err, double *b_other, int32_t *n_other);

/* Stage input of an explicit Runge-Kutta step (reference runge_kutta.py:258-262):
 *   y_out[b,f] = fma(dt[b], sum_{j<n_terms} a[j] * k[j,b,f], y0[b,f])   (the sum is a chain of fma)
 *   t_out[b]   = fma(c, dt[b], t0[b])                                   (skipped if t_out is NULL)
 * k is [n_stages_total, B, F]; only its first n_terms slices are read. */
int tode_erk_stage(int32_t dtype, int64_t batch, int32_t n_features, int32_t n_terms, const double *a, double c,
                   const void *t0, const void *dt, const void *y0, const void *k, void *y_out, void *t_out, void *stream);

/* Weighted stage sum (reference runge_kutta.py:264-267, einsum "b,s,sbf->bf"):
 *   out[b,f] = sum_{s<n_stages} (dt[b] * w[s]) * k[s,b,f]   (+ y0[b,f] when y0 is not NULL)
 * used for the error estimate (w = b_err) and for y1 of methods whose last stage is not the solution. */
int tode_erk_combine(int32_t dtype, int64_t batch, int32_t n_features, int32_t n_stages, const double *w, const void *dt,
                     const void *k, const void *y0, void *out, void *stream);

/* out[b,f] = |err[b,f]| / (atol + rtol * max(|y0[b,f]|, |y1[b,f]|))   (reference step_size_controllers.py:389-393, 734-738);
 * atol and rtol are rounded to float32 first, as the reference's buffers are. */
int tode_error_scale(int32_t dtype, int64_t batch, int32_t n_features, double atol, double rtol, const void *y0, const void *y1,
                     const void *err, void *out, void *stream);

/* Row norms of x [B,F] -> out [B]: TODE_NORM_RMS or TODE_NORM_MAX (reference step_size_controllers.py:170-186). */
int tode_row_norm(int32_t dtype, int32_t norm, int64_t batch, int32_t n_features, const void *x, void *out, void *stream);

/* From the error norm to the decision (reference step_size_controllers.py:394-429, 739-774, dt_factor :289-294, :598-621,
 * PID update_state :640-671):  ratio = max(norm, 1e-38); accept = ratio < 1; dt_next = dt * clamp(factor);
 * status = INFINITE_NORM if ratio is not finite, REACHED_DT_MIN if |dt_next| < dt_min; dt_min/dt_max applied.
 * PID: prev / prev_prev are the history in (NULL for the integral controller), prev_out / prev_prev_out the history
 * after update_state (shifted where accept).  accept is one byte per sample, status int64. */
int tode_control(int32_t dtype, const tode_controller *c, int32_t method_order, int64_t batch, const void *norm, const void *dt,
                 const void *prev, const void *prev_prev, uint8_t *accept, void *dt_next, void *ratio, int64_t *status,
                 void *prev_out, void *prev_prev_out, void *stream);

/* tode_error_scale + tode_row_norm + tode_control in one kernel: {Integral,PID}Controller.adapt_step_size
 * with a built-in norm (reference step_size_controllers.py:370-429, 715-774). */
int tode_adapt_step(int32_t dtype, const tode_controller *c, int32_t method_order, int32_t norm, int64_t batch, int32_t n_features,
                    const void *dt, const void *y0, const void *y1, const void *err, const void *prev, const void *prev_prev,
                    uint8_t *accept, void *dt_next, void *ratio, int64_t *status, void *prev_out, void *prev_prev_out,
                    void *stream);

/* Start step selection, first half (reference step_size_controllers.py:459-479, 804-824): from f0 = f(t_start, y0)
 *   h0[b], y1 = y0 + direction * h0 * f0 [B,F], t1 = t_start + direction * h0 [B]
 * and second half (:481-490, :826-835) from f1 = f(t1, y1): dt0[b] (signed).  `kind` is the controller kind: the
 * integral controller maps h0 == 0 to d2 = inf, the PID controller does not (:481 against :826). */
int tode_initial_step_a(int32_t dtype, int32_t norm, int64_t batch, int32_t n_features, double atol, double rtol, const void *t_start,
                        const void *t_end, const void *y0, const void *f0, void *h0, void *y1, void *t1, void *stream);
int tode_initial_step_b(int32_t dtype, int32_t kind, int32_t norm, int32_t method_order, int64_t batch, int32_t n_features, double atol,
                        double rtol, const void *t_start, const void *t_end, const void *y0, const void *f0, const void *f1,
                        const void *h0, void *dt0, void *stream);

/* The start step with a user-defined norm, whose evaluations happen between the calls:
 *   out = v * (1 / (atol + rtol * |y_ref|))                                 (tode_tolerance_scale: the norm's argument)
 *   d0 = norm(scale(y0)), d1 = norm(scale(f0))  ->  h0, y1, t1              (tode_initial_step_a_norms)
 *   d2n = norm(scale(f1 - f0))                  ->  dt0                      (tode_initial_step_b_norms)
 * d0, d1, d2n, h0 are [B] in the data type. */
int tode_tolerance_scale(int32_t dtype, int64_t batch, int32_t n_features, double atol, double rtol, const void *y_ref, const void *v,
                         void *out, void *stream);
int tode_initial_step_a_norms(int32_t dtype, int64_t batch, int32_t n_features, const void *t_start, const void *t_end, const void *y0,
                              const void *f0, const void *d0, const void *d1, void *h0, void *y1, void *t1, void *stream);
int tode_initial_step_b_norms(int32_t dtype, int32_t kind, int32_t method_order, int64_t batch, const void *t_start, const void *t_end,
                              const void *h0, const void *d1, const void *d2n, void *dt0, void *stream);

/* Quartic dense-output coefficients of a Dopri5 / Tsit5 step, lowest power first: coeff [5,B,F]
 * (reference tsit5.py:123-139; dopri5.py:53-60 -> interpolation.py:138-170).  k is [7,B,F]. */
int tode_quartic_build(int32_t dtype, int32_t method, int64_t batch, int32_t n_features, const void *dt, const void *y0,
                       const void *y1, const void *k, void *coeff, void *stream);

/* The same quartic from a given mid-point value y_mid = y(t0 + dt/2) and the first / last stage derivatives
 * (reference FourthOrderPolynomialInterpolation.from_k, interpolation.py:138-170): coeff [5,B,F]. */
int tode_quartic_from_mid(int32_t dtype, int64_t batch, int32_t n_features, const void *dt, const void *y0, const void *y1,
                          const void *k_first, const void *k_last, const void *y_mid, void *coeff, void *stream);

/* Hermite cubic from the end points and end-point derivatives (reference ThirdOrderPolynomialInterpolation.from_k,
 * interpolation.py:84-106): coeff [4,B,F], lowest power first. */
int tode_cubic_build(int32_t dtype, int64_t batch, int32_t n_features, const void *dt, const void *y0, const void *y1,
                     const void *k_first, const void *k_last, void *coeff, void *stream);

/* Polynomial evaluation (reference interpolation.py:8-40, 103-106, 172-175): for n = 0..count-1, b = idx[n],
 *   x = (t[n] - t0[b]) / (t1[b] - t0[b])  (denominator 1 where it is 0);  out[n,f] = Horner(coeff[degree..0, b, f], x)
 * coeff is [degree+1,B,F], degree in 1..4.  With span_is_dt != 0 the operand `t1` holds the step size and is the
 * denominator as it stands, as in the reference's LinearInterpolation (interpolation.py:56-58), which keeps dt where
 * the higher-order interpolants keep t1 (interpolation.py:76-77, 132-133). */
int tode_poly_eval(int32_t dtype, int32_t degree, int32_t span_is_dt, int64_t batch, int32_t n_features, int64_t count,
                   const void *coeff, const void *t0, const void *t1, const void *t, const int64_t *idx, void *out,
                   void *stream);

/* The same evaluation for every set entry of a [B,E] byte mask, written to ys[b,e,:]
 * (reference adjoints.py:227-233 without materialising the index list). */
int tode_poly_eval_masked(int32_t dtype, int32_t degree, int32_t span_is_dt, int64_t batch, int32_t n_features,
                          int32_t n_eval, const void *coeff, const void *t0, const void *t1, const void *t_eval,
                          const uint8_t *mask, void *ys, void *stream);

/* out[b,:] = mask[b] ? a[b,:] : b[b,:] for rows of `width` values (merge_states, reference runge_kutta.py:216-224,
 * step_size_controllers.py:628-638). */
int tode_select_rows(int32_t dtype, int64_t batch, int32_t width, const uint8_t *mask, const void *a, const void *b, void *out,
                     void *stream);

/*
 * Bookkeeping of one loop iteration (reference adjoints.py:150-255) in one call.
 * Given the step's proposal (y_new, accept, dt_next, optional status of method and controller) it computes
 *   to_update = accept & running;  t, y where to_update;  n_steps += running;  n_accepted += to_update;
 *   running_out = direction * (t_out - t_end) < 0;  status (max of the two, REACHED_MAX_STEPS at max_steps);
 *   to_evaluate[b,e] = pending[b,e] & (direction * (t_out - t_eval[b,e]) >= 0), pending ^= to_evaluate;
 *   dt_out = clamp(running_out ? dt_next : dt, t_min - t_out, t_max - t_out)
 * and the flag block {any sample running, any status != SUCCESS, number of set to_evaluate entries}.
 * Outputs never alias inputs (callers of the protocols may keep earlier t / y / dt tensors).
 * n_steps, n_accepted and pending are updated in place.
 */
enum { TODE_LOOP_ANY_RUNNING = 0, TODE_LOOP_ANY_FAILURE = 1, TODE_LOOP_N_TO_EVALUATE = 2, TODE_LOOP_FLAG_WORDS = 4 };
typedef struct tode_loop_args {
    int32_t dtype, n_features, n_eval, reserved;
    int64_t batch;
    int64_t max_steps;            /* < 0: none */
    const void *t_start, *t_end;  /* [B] */
    const void *t_eval;           /* [B,E] or NULL */
    const void *t, *dt, *y;       /* state before the step: [B], [B], [B,F] */
    const uint8_t *running;       /* [B] */
    const void *y_new;            /* [B,F] step result */
    const uint8_t *accept;        /* [B] */
    const void *dt_next;          /* [B] */
    const int64_t *method_status, *controller_status; /* [B] or NULL */
    void *t_out, *dt_out, *y_out; /* state after the step */
    uint8_t *running_out, *to_update; /* [B] */
    int64_t *status;              /* [B] */
    int64_t *n_steps, *n_accepted; /* [B], in place */
    uint8_t *pending;             /* [B,E], in place, or NULL */
    uint8_t *to_evaluate;         /* [B,E] or NULL */
    int32_t *flags;               /* [TODE_LOOP_FLAG_WORDS] */
} tode_loop_args;
int tode_loop_advance(const tode_loop_args *a, void *stream);

/* Start of the loop (reference adjoints.py:76-79, 107, 121-126): pending[b,e] = 1; where t_eval[b,0] == t_start[b]
 * ys[b,0,:] = y0[b,:] and pending[b,0] = 0; dt_out = clamp(dt, t_min - t_start, t_max - t_start). */
int tode_loop_begin(int32_t dtype, int64_t batch, int32_t n_features, int32_t n_eval, const void *t_start, const void *t_end,
                    const void *t_eval, const void *y0, const void *dt, void *dt_out, uint8_t *pending, void *ys, void *stream);

/* n_initialized[b] = number of leading zeros of pending[b,:] (reference adjoints.py:284-292). */
int tode_count_initialized(int64_t batch, int32_t n_eval, const uint8_t *pending, int64_t *n_initialized, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TORCHODE_AMD_H */
