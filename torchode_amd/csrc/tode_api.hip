// extern "C" surface of libtorchode_amd: argument validation, error reporting
// and the small finalisation kernel.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include "../../include/torchode_amd.h"
#include "tode_internal.h"

namespace tode {

static thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t err, const char *what) {
    if (err == hipSuccess) return TODE_OK;
    return fail(TODE_E_HIP, "%s: %s", what, hipGetErrorString(err));
}

static thread_local int g_fast_variant = 0;
static thread_local bool g_timing = false;
static thread_local bool g_timed = false;
static thread_local hipEvent_t g_ev[2] = {nullptr, nullptr};

static thread_local const char *g_kernel_name = "";

void timing_before(hipStream_t s, const char *kernel_name) {
    g_kernel_name = kernel_name;
    if (!g_timing) return;
    if (!g_ev[0]) {
        (void)hipEventCreate(&g_ev[0]);
        (void)hipEventCreate(&g_ev[1]);
    }
    (void)hipEventRecord(g_ev[0], s);
}

void timing_after(hipStream_t s) {
    if (!g_timing) return;
    (void)hipEventRecord(g_ev[1], s);
    g_timed = true;
}

template <typename T>
__global__ void finalize_kernel(long long batch, int last_iteration, const int32_t *n_steps, const int32_t *n_accepted,
                                const int32_t *n_initialized, const int32_t *status_last, const int32_t *status_idle,
                                int64_t *o_steps, int64_t *o_acc, int64_t *o_init, int64_t *o_status, int n_features,
                                int n_eval, T *ys, const T *y_idle) {
    const long long b = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= batch) return;
    const int ns = n_steps[b];
    const bool at_last = ns == last_iteration;
    o_steps[b] = ns;
    o_acc[b] = n_accepted[b];
    o_init[b] = n_initialized[b];
    o_status[b] = at_last ? status_last[b] : status_idle[b];
    if (n_eval == 0 && !at_last) {
        for (int f = 0; f < n_features; ++f) ys[b * n_features + f] = y_idle[b * n_features + f];
    }
}

}  // namespace tode

extern "C" {

int tode_abi_version(void) { return TODE_ABI_VERSION; }

const char *tode_last_error(void) { return tode::g_error; }

int tode_set_fast_kernel_variant(int variant) {
    if (variant < 0 || variant > 2) return tode::fail(TODE_E_INVALID, "variant must be 0 (auto), 1 (one wavefront) or 2 (two wavefronts)");
    tode::g_fast_variant = variant;
    return TODE_OK;
}

int tode_set_kernel_timing(int enable) {
    tode::g_timing = enable != 0;
    if (!enable) tode::g_timed = false;
    return TODE_OK;
}

const char *tode_last_solve_kernel_name(void) { return tode::g_kernel_name; }

int tode_last_solve_kernel_ms(float *out_ms) {
    using namespace tode;
    if (!out_ms) return fail(TODE_E_INVALID, "null output pointer");
    if (!g_timing || !g_timed) return fail(TODE_E_INVALID, "kernel timing is off or no solve was launched");
    int rc = check_hip(hipEventSynchronize(g_ev[1]), "hipEventSynchronize");
    if (rc) return rc;
    return check_hip(hipEventElapsedTime(out_ms, g_ev[0], g_ev[1]), "hipEventElapsedTime");
}

int tode_solve_builtin(const tode_solve_args *a, const tode_controller *c, void *stream) {
    using namespace tode;
    if (!a || !c) return fail(TODE_E_INVALID, "null argument struct");
    if (a->batch < 0 || a->n_features <= 0 || a->n_eval < 0 || a->n_params < 0)
        return fail(TODE_E_INVALID, "bad sizes: batch=%lld F=%d E=%d P=%d", (long long)a->batch, a->n_features, a->n_eval, a->n_params);
    if (a->batch > 0 && (!a->y0 || !a->t_start || !a->t_end || !a->ys || (a->n_params > 0 && !a->params)))
        return fail(TODE_E_INVALID, "null problem pointer");
    if (a->t_start_stride < 1 || a->t_end_stride < 1)
        return fail(TODE_E_INVALID, "t_start_stride / t_end_stride must be >= 1 (got %lld, %lld)", (long long)a->t_start_stride, (long long)a->t_end_stride);
    if (a->n_eval > 0 && a->batch > 0 && !a->t_eval) return fail(TODE_E_INVALID, "n_eval > 0 but t_eval is null");
    if (a->n_eval == 0 && a->batch > 0 && !a->y_idle) return fail(TODE_E_INVALID, "n_eval == 0 needs y_idle");
    if (!a->flags || (a->batch > 0 && (!a->n_steps || !a->n_accepted || !a->n_initialized || !a->status_last || !a->status_idle)))
        return fail(TODE_E_INVALID, "null output pointer");
    if (c->kind != TODE_CTRL_INTEGRAL && c->kind != TODE_CTRL_PID) return fail(TODE_E_INVALID, "unknown controller kind %d", c->kind);
    if (a->batch > (int64_t)2147483647 * TODE_BLOCK) return fail(TODE_E_UNSUPPORTED, "batch too large");
    hipStream_t s = (hipStream_t)stream;
    if (a->dtype == TODE_F32) return solve_builtin_f32(*a, *c, s);
    if (a->dtype == TODE_F64) return solve_builtin_f64(*a, *c, s);
    return fail(TODE_E_INVALID, "unknown dtype %d", a->dtype);
}

int tode_solve_builtin_fast(const tode_solve_args *a, const tode_controller *c, int64_t *ns, int64_t *na, int64_t *ni,
                            int64_t *st, void *stream) {
    using namespace tode;
    if (!a || !c) return fail(TODE_E_INVALID, "null argument struct");
    if (a->batch < 0 || a->n_features <= 0 || a->n_eval < 0 || a->n_params < 0)
        return fail(TODE_E_INVALID, "bad sizes: batch=%lld F=%d E=%d P=%d", (long long)a->batch, a->n_features, a->n_eval, a->n_params);
    if (a->n_eval == 0) return fail(TODE_E_UNSUPPORTED, "the fast entry point needs evaluation points");
    if (c->has_dt_min || c->has_dt_max) return fail(TODE_E_UNSUPPORTED, "the fast entry point does not take dt_min / dt_max");
    if (c->kind != TODE_CTRL_INTEGRAL && c->kind != TODE_CTRL_PID) return fail(TODE_E_INVALID, "unknown controller kind %d", c->kind);
    if (!a->flags) return fail(TODE_E_INVALID, "null flags pointer");
    if (a->batch > 0 && (!a->y0 || !a->t_start || !a->t_end || !a->t_eval || !a->ys || (a->n_params > 0 && !a->params) || !ns || !na || !ni || !st))
        return fail(TODE_E_INVALID, "null pointer");
    if (a->t_start_stride < 1 || a->t_end_stride < 1)
        return fail(TODE_E_INVALID, "t_start_stride / t_end_stride must be >= 1 (got %lld, %lld)", (long long)a->t_start_stride, (long long)a->t_end_stride);
    if (a->batch > (int64_t)2147483647 * 64) return fail(TODE_E_UNSUPPORTED, "batch too large");
    hipStream_t s = (hipStream_t)stream;
    if (a->dtype != TODE_F32 && a->dtype != TODE_F64) return fail(TODE_E_INVALID, "unknown dtype %d", a->dtype);
    if (a->term == TODE_TERM_REACTION_DIFFUSION) {
        if (a->dtype != TODE_F32) return fail(TODE_E_UNSUPPORTED, "the grid kernel is built for float32");
        return solve_grid_f32(*a, *c, ns, na, ni, st, s);
    }
    if (a->term == TODE_TERM_MLP) {
        if (a->dtype != TODE_F32) return fail(TODE_E_UNSUPPORTED, "the MLP kernel is built for float32");
        return solve_mlp_f32(*a, *c, ns, na, ni, st, s);
    }
    if (g_fast_variant != 1) {
        // small batches: two wavefronts per group of 64 samples (stepper + dense-output evaluator)
        bool used = false;
        int rc = a->dtype == TODE_F32 ? solve_pair_f32(*a, *c, ns, na, ni, st, s, &used) : solve_pair_f64(*a, *c, ns, na, ni, st, s, &used);
        if (rc || used) return rc;
        if (g_fast_variant == 2) return fail(TODE_E_UNSUPPORTED, "the two-wavefront kernel does not cover this problem size");
    }
    if (a->dtype == TODE_F32) return solve_fast_f32(*a, *c, ns, na, ni, st, s);
    return solve_fast_f64(*a, *c, ns, na, ni, st, s);
}

int tode_finalize_stats(int64_t batch, int64_t last_iteration, const int32_t *n_steps, const int32_t *n_accepted,
                        const int32_t *n_initialized, const int32_t *status_last, const int32_t *status_idle,
                        int64_t *out_n_steps, int64_t *out_n_accepted, int64_t *out_n_initialized, int64_t *out_status,
                        int32_t dtype, int32_t n_features, int32_t n_eval, void *ys, const void *y_idle, void *stream) {
    using namespace tode;
    if (batch < 0) return fail(TODE_E_INVALID, "negative batch");
    if (batch == 0) return TODE_OK;
    if (!n_steps || !n_accepted || !n_initialized || !status_last || !status_idle || !out_n_steps || !out_n_accepted ||
        !out_n_initialized || !out_status)
        return fail(TODE_E_INVALID, "null pointer");
    if (n_eval == 0 && (!ys || !y_idle)) return fail(TODE_E_INVALID, "n_eval == 0 needs ys and y_idle");
    hipStream_t s = (hipStream_t)stream;
    const unsigned blocks = (unsigned)((batch + 255) / 256);
    if (dtype == TODE_F32)
        hipLaunchKernelGGL(finalize_kernel<float>, dim3(blocks), dim3(256), 0, s, (long long)batch, (int)last_iteration, n_steps,
                           n_accepted, n_initialized, status_last, status_idle, out_n_steps, out_n_accepted, out_n_initialized,
                           out_status, n_features, n_eval, (float *)ys, (const float *)y_idle);
    else if (dtype == TODE_F64)
        hipLaunchKernelGGL(finalize_kernel<double>, dim3(blocks), dim3(256), 0, s, (long long)batch, (int)last_iteration, n_steps,
                           n_accepted, n_initialized, status_last, status_idle, out_n_steps, out_n_accepted, out_n_initialized,
                           out_status, n_features, n_eval, (double *)ys, (const double *)y_idle);
    else
        return fail(TODE_E_INVALID, "unknown dtype %d", dtype);
    return check_hip(hipGetLastError(), "tode_finalize_stats launch");
}

}  // extern "C"
