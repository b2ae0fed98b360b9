// extern "C" surface of libtorchode_amd: argument validation, error reporting
// and the small finalisation kernel.
#include <hip/hip_runtime.h>
#include <limits.h>
#include <stdarg.h>
#include <stdio.h>

#include <atomic>
#include <mutex>

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

// ---- flag slots of tode_solve_builtin_fast_sync -------------------------------------------------
// Per device: FLAG_SLOTS blocks of FLAG_SLOT_WORDS int32 in device memory (four flag words at their
// start values and a count of finished workgroups, put back by the kernel that used them) and as
// many in pinned, coherent host memory (the published flags and a sequence number).  A call takes a
// free slot, so calls from several host threads or on several streams do not share words.
constexpr int FLAG_SLOTS = 64, FLAG_SLOT_WORDS = 8, FLAG_DEVICES = 64;

struct FlagPool {
    int32_t *dev = nullptr;
    int32_t *host = nullptr;
    int32_t *host_as_seen_by_device = nullptr;
    std::atomic<int> busy[FLAG_SLOTS];
    int32_t sequence[FLAG_SLOTS];
    std::atomic<unsigned> next;
};
static FlagPool g_flag_pools[FLAG_DEVICES];  // static storage: zero-initialised
static std::mutex g_flag_mutex;
static thread_local const FlagTarget *g_flag_target = nullptr;

const FlagTarget *flag_target() { return g_flag_target; }

static int flag_pool(hipStream_t s, FlagPool **out) {
    int device = 0;
    int rc = check_hip(s ? hipStreamGetDevice(s, &device) : hipGetDevice(&device), "device of the stream");
    if (rc) return rc;
    if (device < 0 || device >= FLAG_DEVICES) return fail(TODE_E_UNSUPPORTED, "device index %d", device);
    FlagPool &pool = g_flag_pools[device];
    std::lock_guard<std::mutex> lock(g_flag_mutex);
    if (!pool.dev) {
        int current = 0;
        if ((rc = check_hip(hipGetDevice(&current), "hipGetDevice"))) return rc;
        if (current != device && (rc = check_hip(hipSetDevice(device), "hipSetDevice"))) return rc;
        const size_t bytes = (size_t)FLAG_SLOTS * FLAG_SLOT_WORDS * sizeof(int32_t);
        int32_t start[FLAG_SLOTS * FLAG_SLOT_WORDS] = {};
        for (int i = 0; i < FLAG_SLOTS; ++i) start[i * FLAG_SLOT_WORDS + TODE_FLAG_FIRST_FAILURE] = INT_MAX;
        int32_t *dev = nullptr, *host = nullptr, *host_dev = nullptr;
        hipError_t err = hipMalloc((void **)&dev, bytes);
        if (err == hipSuccess) err = hipMemcpy(dev, start, bytes, hipMemcpyHostToDevice);
        if (err == hipSuccess) err = hipHostMalloc((void **)&host, bytes, hipHostMallocPortable | hipHostMallocMapped | hipHostMallocCoherent);
        if (err == hipSuccess) err = hipHostGetDevicePointer((void **)&host_dev, host, 0);
        if (current != device) (void)hipSetDevice(current);
        if (err != hipSuccess) {
            if (dev) (void)hipFree(dev);
            if (host) (void)hipHostFree(host);
            return check_hip(err, "allocating the flag slots");
        }
        for (int i = 0; i < FLAG_SLOTS * FLAG_SLOT_WORDS; ++i) host[i] = 0;
        pool.host = host;
        pool.host_as_seen_by_device = host_dev;
        pool.dev = dev;
    }
    *out = &pool;
    return TODE_OK;
}

// Spins on the slot's sequence word; looks at the stream now and then, so that a kernel that never
// ran (or a failed device) ends the wait with an error instead of a hang.
static int wait_for_flags(const int32_t *slot, int32_t sequence, hipStream_t s) {
    for (unsigned spin = 1;; ++spin) {
        if (__atomic_load_n(&slot[TODE_FLAG_WORDS], __ATOMIC_ACQUIRE) == sequence) return TODE_OK;
        if ((spin & 0x3FFF) == 0) {
            const hipError_t q = hipStreamQuery(s);
            if (q == hipSuccess) {
                if (__atomic_load_n(&slot[TODE_FLAG_WORDS], __ATOMIC_ACQUIRE) == sequence) return TODE_OK;
                return fail(TODE_E_HIP, "the stream is idle but the solve kernel has not published its flags");
            }
            if (q != hipErrorNotReady) return check_hip(q, "hipStreamQuery while waiting for the solve kernel");
        }
        __builtin_ia32_pause();
    }
}

// ---- static scratch of tode_solve_builtin_fast_static -------------------------------------------
// Device memory that belongs to the loaded code object, one copy per GPU, held until the process
// ends: the working flag words of a solve (four flags and the count of finished workgroups) in the
// first STATIC_FLAG_BYTES, behind them the staging area for the final states of a solve without
// evaluation points.  Host code never uses the array's name as an address: static_scratch() asks the
// runtime for the device's copy once and keeps the pointer.
constexpr size_t STATIC_FLAG_BYTES = 256;
static __device__ __align__(256) unsigned char scratch[STATIC_FLAG_BYTES + TODE_STATIC_STAGING_BYTES];
static void *g_scratch_ptr[FLAG_DEVICES];  // static storage: null until asked for
static std::mutex g_scratch_mutex;
// Who used a device's array last: a call on another stream is refused while that work has not finished (the event
// behind it has not fired).  The event is made with the array's address, on the first call on the device.
struct StaticUse {
    hipEvent_t done = nullptr;
    hipStream_t stream = nullptr;
    bool recorded = false;
};
static StaticUse g_static_use[FLAG_DEVICES];

// (called with g_scratch_mutex held)
static int static_scratch(hipStream_t s, unsigned char **out, int *device_out) {
    int device = 0;
    int rc = check_hip(s ? hipStreamGetDevice(s, &device) : hipGetDevice(&device), "device of the stream");
    if (rc) return rc;
    if (device < 0 || device >= FLAG_DEVICES) return fail(TODE_E_UNSUPPORTED, "device index %d", device);
    *device_out = device;
    if (!g_scratch_ptr[device]) {
        int current = 0;
        if ((rc = check_hip(hipGetDevice(&current), "hipGetDevice"))) return rc;
        if (current != device && (rc = check_hip(hipSetDevice(device), "hipSetDevice"))) return rc;
        void *ptr = nullptr;
        hipError_t err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        hipEvent_t done = nullptr;
        if (err == hipSuccess && ptr) err = hipEventCreateWithFlags(&done, hipEventDisableTiming);
        if (current != device) (void)hipSetDevice(current);
        if (err != hipSuccess) return check_hip(err, "hipGetSymbolAddress of the static scratch array");
        if (!ptr) return fail(TODE_E_HIP, "hipGetSymbolAddress returned a null address for the static scratch array");
        g_static_use[device].done = done;
        g_scratch_ptr[device] = ptr;
    }
    *out = (unsigned char *)g_scratch_ptr[device];
    return TODE_OK;
}

// The working flag words at their start values, whatever the last call left there.
static __global__ void static_flags_reset_kernel(int32_t *flags) {
    if (threadIdx.x <= TODE_FLAG_WORDS) flags[threadIdx.x] = threadIdx.x == TODE_FLAG_FIRST_FAILURE ? INT_MAX : 0;
}

// Flags of a solve that launched no solve kernel (an empty batch).
static __global__ void empty_flags_kernel(int32_t *flags_out) {
    if (threadIdx.x < TODE_FLAG_WORDS) flags_out[threadIdx.x] = threadIdx.x == TODE_FLAG_FIRST_FAILURE ? INT_MAX : 0;
}

// select_end_point_kernel with the loop's iteration count read from the published flag block
// instead of passed by the host; does nothing when the batch left the common case.
template <typename T>
__global__ void select_end_point_by_flags_kernel(long long n, int F, const int32_t *flags, const int64_t *n_steps, T *ys, const T *y_idle) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n || flags[TODE_FLAG_NEEDS_GENERAL] != 0) return;
    if (n_steps[i / F] < (long long)flags[TODE_FLAG_MAX_ITERATIONS]) ys[i] = y_idle[i];
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

template <typename T>
__global__ void select_end_point_kernel(long long n, int F, long long last, const int64_t *n_steps, T *ys, const T *y_idle) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && n_steps[i / F] < last) ys[i] = y_idle[i];
}

}  // namespace tode

extern "C" {

int tode_abi_version(void) { return TODE_ABI_VERSION; }

#ifndef TODE_SOURCE_HASH
#define TODE_SOURCE_HASH ""
#endif
const char *tode_source_hash(void) { return TODE_SOURCE_HASH; }

const char *tode_last_error(void) { return tode::g_error; }

int tode_set_fast_kernel_variant(int variant) {
    if (variant < 0 || variant > 2) return tode::fail(TODE_E_INVALID, "variant must be 0 (automatic), 1 (one wavefront per 64 samples) or 2 (two wavefronts)");
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
    if (!known_dtype(a->dtype)) return fail(TODE_E_INVALID, "unknown dtype %d", a->dtype);
    const int data = data_type(a->dtype), time = time_type(a->dtype);
    if (a->record) {  // the same kernel, keeping the loop state of every iteration
        if (data == time) return data == TODE_F32 ? solve_builtin_f32_record(*a, *c, s) : solve_builtin_f64_record(*a, *c, s);
        return data == TODE_F32 ? solve_builtin_t64_y32_record(*a, *c, s) : solve_builtin_t32_y64_record(*a, *c, s);
    }
    if (data == time) return data == TODE_F32 ? solve_builtin_f32(*a, *c, s) : solve_builtin_f64(*a, *c, s);
    return data == TODE_F32 ? solve_builtin_t64_y32(*a, *c, s) : solve_builtin_t32_y64(*a, *c, s);
}

int tode_solve_builtin_fast(const tode_solve_args *a, const tode_controller *c, int64_t *ns, int64_t *na, int64_t *ni,
                            int64_t *st, void *stream) {
    using namespace tode;
    if (!a || !c) return fail(TODE_E_INVALID, "null argument struct");
    if (a->batch < 0 || a->n_features <= 0 || a->n_eval < 0 || a->n_params < 0)
        return fail(TODE_E_INVALID, "bad sizes: batch=%lld F=%d E=%d P=%d", (long long)a->batch, a->n_features, a->n_eval, a->n_params);
    const bool end_only = a->n_eval == 0;
    if (end_only && a->batch > 0 && !a->y_idle) return fail(TODE_E_INVALID, "n_eval == 0 needs y_idle");
    if (c->has_dt_min || c->has_dt_max) return fail(TODE_E_UNSUPPORTED, "the fast entry point does not take dt_min / dt_max");
    if (c->kind != TODE_CTRL_INTEGRAL && c->kind != TODE_CTRL_PID) return fail(TODE_E_INVALID, "unknown controller kind %d", c->kind);
    if (!a->flags) return fail(TODE_E_INVALID, "null flags pointer");
    if (a->batch > 0 && (!a->y0 || !a->t_start || !a->t_end || (!end_only && !a->t_eval) || !a->ys || (a->n_params > 0 && !a->params) || !ns || !na || !ni || !st))
        return fail(TODE_E_INVALID, "null pointer");
    if (a->t_start_stride < 1 || a->t_end_stride < 1)
        return fail(TODE_E_INVALID, "t_start_stride / t_end_stride must be >= 1 (got %lld, %lld)", (long long)a->t_start_stride, (long long)a->t_end_stride);
    if (a->batch > (int64_t)2147483647 * 64) return fail(TODE_E_UNSUPPORTED, "batch too large");
    hipStream_t s = (hipStream_t)stream;
    if (!known_dtype(a->dtype)) return fail(TODE_E_INVALID, "unknown dtype %d", a->dtype);
    if (a->dtype & TODE_DTYPE_PAIR) return fail(TODE_E_UNSUPPORTED, "the fast entry point is built for time and data in one dtype");
    if (a->record && (a->term == TODE_TERM_REACTION_DIFFUSION || a->term == TODE_TERM_MLP))
        return fail(TODE_E_UNSUPPORTED, "a record of the loop state is written for the small systems only");
    if (a->term == TODE_TERM_REACTION_DIFFUSION) {
        return a->dtype == TODE_F32 ? solve_grid_f32(*a, *c, ns, na, ni, st, s) : solve_grid_f64(*a, *c, ns, na, ni, st, s);
    }
    if (a->term == TODE_TERM_MLP) {
        if (a->dtype != TODE_F32) return fail(TODE_E_UNSUPPORTED, "the MLP kernel is built for float32");
        return solve_mlp_f32(*a, *c, ns, na, ni, st, s);
    }
    if (a->record) {  // the solve and the record of its loop state in one kernel: the stepper of the two-wavefront kernel
                      // writes it for small batches, the single-wavefront kernel otherwise
        if (end_only) return fail(TODE_E_UNSUPPORTED, "a record from the fast entry point needs evaluation points");
        if (g_fast_variant == 0 || g_fast_variant == 2) {
            bool used = false;
            int rc = a->dtype == TODE_F32 ? solve_pair_f32_record(*a, *c, ns, na, ni, st, s, &used) : solve_pair_f64_record(*a, *c, ns, na, ni, st, s, &used);
            if (rc || used) return rc;
            if (g_fast_variant == 2) return fail(TODE_E_UNSUPPORTED, "the two-wavefront kernel does not cover this problem size");
        }
        return a->dtype == TODE_F32 ? solve_fast_f32_record(*a, *c, ns, na, ni, st, s) : solve_fast_f64_record(*a, *c, ns, na, ni, st, s);
    }
    if (g_fast_variant == 0 || g_fast_variant == 2) {
        // small batches: two wavefronts per group of 64 samples (stepper + dense-output evaluator)
        bool used = false;
        int rc = a->dtype == TODE_F32 ? solve_pair_f32(*a, *c, ns, na, ni, st, s, &used) : solve_pair_f64(*a, *c, ns, na, ni, st, s, &used);
        if (rc || used) return rc;
        if (g_fast_variant == 2) return fail(TODE_E_UNSUPPORTED, "the two-wavefront kernel does not cover this problem size");
    }
    if (end_only)
        return fail(TODE_E_UNSUPPORTED, "without evaluation points the fast entry point covers batches of up to %d samples", TODE_END_ONLY_MAX_BATCH);
    if (a->dtype == TODE_F32) return solve_fast_f32(*a, *c, ns, na, ni, st, s);
    return solve_fast_f64(*a, *c, ns, na, ni, st, s);
}

int tode_mlp_pack_weights(const void *raw, int64_t n_raw, int32_t matrix_inputs, void *packed, void *stream) {
    return tode::mlp_pack_weights((const float *)raw, (long long)n_raw, 64, matrix_inputs, (float *)packed, (hipStream_t)stream);
}

int tode_mlp_pack_weights_for(const void *raw, int64_t n_raw, int32_t n_features, int32_t matrix_inputs, void *packed, void *stream) {
    return tode::mlp_pack_weights((const float *)raw, (long long)n_raw, n_features, matrix_inputs, (float *)packed, (hipStream_t)stream);
}

int tode_solve_builtin_fast_sync(const tode_solve_args *a, const tode_controller *c, int64_t *ns, int64_t *na, int64_t *ni,
                                 int64_t *st, void *stream, int32_t *flags_out) {
    using namespace tode;
    if (!a || !c || !flags_out) return fail(TODE_E_INVALID, "null argument");
    hipStream_t s = (hipStream_t)stream;
    FlagPool *pool = nullptr;
    int rc = flag_pool(s, &pool);
    if (rc) return rc;
    int slot = -1;
    const unsigned first = pool->next.fetch_add(1, std::memory_order_relaxed);
    for (int i = 0; i < FLAG_SLOTS && slot < 0; ++i) {
        const int candidate = (int)((first + i) % FLAG_SLOTS);
        if (pool->busy[candidate].exchange(1, std::memory_order_acquire) == 0) slot = candidate;
    }
    if (slot < 0) return fail(TODE_E_UNSUPPORTED, "all %d flag slots of this device are in use by calls that have not returned", FLAG_SLOTS);

    // sequence numbers 1, 2, ... INT_MAX, 1, ...: never the 0 the host words start with
    const int32_t sequence = pool->sequence[slot] = pool->sequence[slot] == INT_MAX ? 1 : pool->sequence[slot] + 1;
    const FlagTarget target = {pool->dev + slot * FLAG_SLOT_WORDS, pool->host_as_seen_by_device + slot * FLAG_SLOT_WORDS, sequence};
    tode_solve_args b = *a;
    b.flags = target.dev;
    g_flag_target = &target;
    rc = tode_solve_builtin_fast(&b, c, ns, na, ni, st, stream);
    g_flag_target = nullptr;
    if (rc == TODE_E_UNSUPPORTED && (a->n_eval > 0 || a->y_idle) && !c->has_dt_min && !c->has_dt_max &&
        a->term != TODE_TERM_REACTION_DIFFUSION && a->term != TODE_TERM_MLP) {
        // a small system in a shape the fast kernels do not take (no evaluation points, or very many of them, in a
        // batch too large for the two-wavefront kernel) or with a controller exponent that is not computed through pow:
        // no solve kernel was launched, and the caller is sent to the general kernel like any batch that leaves the
        // common case
        flags_out[TODE_FLAG_MAX_ITERATIONS] = 0;
        flags_out[TODE_FLAG_FIRST_FAILURE] = INT_MAX;
        flags_out[TODE_FLAG_NON_MONOTONE] = 0;
        flags_out[TODE_FLAG_NEEDS_GENERAL] = 1;
        rc = TODE_OK;
    } else if (rc == TODE_OK && a->batch == 0) {  // nothing was launched
        flags_out[TODE_FLAG_MAX_ITERATIONS] = 0;
        flags_out[TODE_FLAG_FIRST_FAILURE] = INT_MAX;
        flags_out[TODE_FLAG_NON_MONOTONE] = flags_out[TODE_FLAG_NEEDS_GENERAL] = 0;
    } else if (rc == TODE_OK) {
        const int32_t *host = pool->host + slot * FLAG_SLOT_WORDS;
        rc = wait_for_flags(host, sequence, s);
        if (rc == TODE_OK)
            for (int i = 0; i < TODE_FLAG_WORDS; ++i) flags_out[i] = host[i];
        if (rc == TODE_OK && a->n_eval == 0 && !flags_out[TODE_FLAG_NEEDS_GENERAL])
            rc = tode_select_end_point(a->batch, a->n_features, a->dtype, flags_out[TODE_FLAG_MAX_ITERATIONS], ns, a->ys, a->y_idle, stream);
    }
    // (after a failed wait the slot's words may be anything: the slot stays out of use)
    if (rc == TODE_OK || rc == TODE_E_INVALID || rc == TODE_E_UNSUPPORTED) pool->busy[slot].store(0, std::memory_order_release);
    return rc;
}

int tode_solve_builtin_fast_static(const tode_solve_args *a, const tode_controller *c, int64_t *ns, int64_t *na, int64_t *ni,
                                   int64_t *st, int32_t *flags_out, void *stream) {
    using namespace tode;
    if (!a || !c || !flags_out) return fail(TODE_E_INVALID, "null argument");
    if (a->batch < 0 || a->n_features <= 0 || a->n_eval < 0) return fail(TODE_E_INVALID, "bad sizes: batch=%lld F=%d E=%d", (long long)a->batch, a->n_features, a->n_eval);
    if (!known_dtype(a->dtype)) return fail(TODE_E_INVALID, "unknown dtype %d", a->dtype);
    if (a->dtype & TODE_DTYPE_PAIR) return fail(TODE_E_UNSUPPORTED, "the fast entry points are built for time and data in one dtype");
    const bool end_only = a->n_eval == 0;
    const size_t value_bytes = a->dtype == TODE_F32 ? 4 : 8;
    if (end_only && (uint64_t)a->batch * (uint64_t)a->n_features > TODE_STATIC_STAGING_BYTES / value_bytes)
        return fail(TODE_E_UNSUPPORTED, "without evaluation points the final states of the batch are staged in the static scratch array: "
                    "%lld x %d values of %zu bytes exceed its %lld bytes", (long long)a->batch, a->n_features, value_bytes, (long long)TODE_STATIC_STAGING_BYTES);
    hipStream_t s = (hipStream_t)stream;
    unsigned char *base = nullptr;
    // One call at a time enqueues work on a device's array (host threads take turns here), and a call on another
    // stream than the last one's is refused while the last one's work is still running: on one stream calls are
    // ordered by the stream, across streams nothing would order them.  A stream under capture launches nothing
    // now, so there is nothing to look at: the owner of the graph keeps its replays apart from other calls.
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    int device = 0;
    int rc = static_scratch(s, &base, &device);
    if (rc) return rc;
    StaticUse &use = g_static_use[device];
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (s && (rc = check_hip(hipStreamIsCapturing(s, &capture), "hipStreamIsCapturing"))) return rc;
    const bool live = capture == hipStreamCaptureStatusNone;
    if (live && use.recorded && use.stream != s) {
        const hipError_t q = hipEventQuery(use.done);
        if (q == hipErrorNotReady)
            return fail(TODE_E_UNSUPPORTED, "the static scratch array of this GPU is in use by a call on another stream that has not finished: "
                        "calls that overlap on one GPU have to be serialised by the caller");
        if (q != hipSuccess) return check_hip(q, "hipEventQuery of the last static call");
    }
    int32_t *words = (int32_t *)base;
    void *staging = base + STATIC_FLAG_BYTES;

    tode_solve_args b = *a;
    b.flags = words;
    if (end_only) b.y_idle = staging;
    const FlagTarget target = {words, flags_out, 0};
    struct MarkUse {  // (whichever way the call leaves from here on: the work enqueued so far is the array's last use)
        StaticUse &use;
        hipStream_t s;
        bool live;
        ~MarkUse() {
            if (live && hipEventRecord(use.done, s) == hipSuccess) use.stream = s, use.recorded = true;
        }
    } mark{use, s, live};
    hipLaunchKernelGGL(static_flags_reset_kernel, dim3(1), dim3(64), 0, s, words);
    g_flag_target = &target;
    rc = tode_solve_builtin_fast(&b, c, ns, na, ni, st, stream);
    g_flag_target = nullptr;
    if (rc) return rc;
    if (a->batch == 0) {
        hipLaunchKernelGGL(empty_flags_kernel, dim3(1), dim3(64), 0, s, flags_out);
        return check_hip(hipGetLastError(), "tode_solve_builtin_fast_static launch");
    }
    if (end_only) {
        const long long n = (long long)a->batch * a->n_features;
        const unsigned blocks = (unsigned)((n + 255) / 256);
        if (a->dtype == TODE_F32)
            hipLaunchKernelGGL(select_end_point_by_flags_kernel<float>, dim3(blocks), dim3(256), 0, s, n, (int)a->n_features, flags_out, ns, (float *)a->ys, (const float *)staging);
        else
            hipLaunchKernelGGL(select_end_point_by_flags_kernel<double>, dim3(blocks), dim3(256), 0, s, n, (int)a->n_features, flags_out, ns, (double *)a->ys, (const double *)staging);
    }
    return check_hip(hipGetLastError(), "tode_solve_builtin_fast_static launch");
}

int tode_select_end_point(int64_t batch, int32_t n_features, int32_t dtype, int64_t last_iteration, const int64_t *n_steps, void *ys,
                          const void *y_idle, void *stream) {
    using namespace tode;
    if (batch < 0 || n_features <= 0) return fail(TODE_E_INVALID, "bad sizes: batch=%lld F=%d", (long long)batch, n_features);
    if (batch == 0) return TODE_OK;
    if (!n_steps || !ys || !y_idle) return fail(TODE_E_INVALID, "null pointer");
    const long long n = (long long)batch * n_features;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TODE_F32)
        hipLaunchKernelGGL(select_end_point_kernel<float>, dim3(blocks), dim3(256), 0, s, n, (int)n_features, (long long)last_iteration, n_steps, (float *)ys, (const float *)y_idle);
    else if (dtype == TODE_F64)
        hipLaunchKernelGGL(select_end_point_kernel<double>, dim3(blocks), dim3(256), 0, s, n, (int)n_features, (long long)last_iteration, n_steps, (double *)ys, (const double *)y_idle);
    else
        return fail(TODE_E_INVALID, "unknown dtype %d", dtype);
    return check_hip(hipGetLastError(), "tode_select_end_point launch");
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

namespace tode {
// Layout of the workspace of tode_solve_builtin_auto: each part starts at a multiple of 256 bytes.
struct Workspace {
    int64_t flags, counters, y_idle, pending, bytes;
};
static Workspace workspace_layout(const tode_solve_args &a) {
    auto up = [](int64_t n) { return (n + 255) / 256 * 256; };
    const int64_t B = a.batch > 0 ? a.batch : 0, elem = data_type(a.dtype) == TODE_F64 ? 8 : 4;
    Workspace w;
    w.flags = 0;
    w.counters = up(TODE_FLAG_WORDS * 4);
    w.y_idle = w.counters + up(5 * B * 4);
    w.pending = w.y_idle + (a.n_eval == 0 ? up(B * a.n_features * elem) : 0);
    w.bytes = w.pending + up(B * a.n_eval);
    return w;
}
}  // namespace tode

int64_t tode_solve_workspace_bytes(const tode_solve_args *a) {
    if (!a || a->n_features <= 0 || a->n_eval < 0) return -1;
    return tode::workspace_layout(*a).bytes;
}

int tode_solve_builtin_auto(const tode_solve_args *a, const tode_controller *c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st,
                            void *workspace, int64_t workspace_bytes, int32_t allow_one_kernel, void *stream, int64_t *iterations) {
    using namespace tode;
    if (!a || !c || !iterations) return fail(TODE_E_INVALID, "null argument");
    if (a->batch < 0 || a->n_features <= 0 || a->n_eval < 0 || a->n_params < 0)
        return fail(TODE_E_INVALID, "bad sizes: batch=%lld F=%d E=%d P=%d", (long long)a->batch, a->n_features, a->n_eval, a->n_params);
    if (!known_dtype(a->dtype)) return fail(TODE_E_INVALID, "unknown dtype %d", a->dtype);
    const bool one_dtype = !(a->dtype & TODE_DTYPE_PAIR);  // (time and data in different types: the general kernel)
    const Workspace w = workspace_layout(*a);
    if (!workspace || workspace_bytes < w.bytes)
        return fail(TODE_E_INVALID, "the workspace holds %lld bytes, this problem needs %lld (tode_solve_workspace_bytes)", (long long)workspace_bytes, (long long)w.bytes);
    if (a->batch > 0 && (!ns || !na || !ni || !st)) return fail(TODE_E_INVALID, "null output pointer");
    hipStream_t s = (hipStream_t)stream;
    unsigned char *ws = (unsigned char *)workspace;
    const int64_t B = a->batch, E = a->n_eval, elem = data_type(a->dtype) == TODE_F64 ? 8 : 4;
    const bool small_system = a->term == TODE_TERM_LINEAR_DECAY || a->term == TODE_TERM_VAN_DER_POL || a->term == TODE_TERM_LORENZ63;

    tode_solve_args b = *a;
    b.iteration_cap = -1;
    b.pending = nullptr;
    b.record = nullptr;
    b.y_idle = E == 0 ? ws + w.y_idle : nullptr;

    // The common case first: one kernel that writes what the reference returns.  It reports through its flag words when the
    // batch needs the general kernel (rows of evaluation points that are not monotone, a non-success status, non-finite values).
    bool one_kernel = one_dtype && !c->has_dt_min && !c->has_dt_max;
    if (small_system) {
        // (no evaluation points, or more than fit on chip: built for batches that leave SIMDs to spare)
        one_kernel = one_kernel && allow_one_kernel && ((E > 0 && E * elem <= 1024) || (B > 0 && B <= TODE_END_ONLY_MAX_BATCH));
    } else {
        if (a->term == TODE_TERM_REACTION_DIFFUSION)
            one_kernel = one_kernel && ((a->n_features == 16 * 16 || a->n_features == 32 * 32 || a->n_features == 64 * 64) ? E <= 8192
                                                                                                                           : (a->n_features == 128 * 128 && a->dtype == TODE_F32 && E <= 4096));
        else if (a->term == TODE_TERM_MLP)
            one_kernel = one_kernel && a->dtype == TODE_F32 && a->n_features >= 1 && a->n_features <= 64 && E <= 512;
        else
            return fail(TODE_E_INVALID, "unknown term %d", a->term);
        if (!one_kernel) return fail(TODE_E_UNSUPPORTED, "no whole-solve kernel for this term in this shape, dtype or controller setting");
    }
    if (one_kernel) {
        int32_t fl[TODE_FLAG_WORDS];
        int rc = tode_solve_builtin_fast_sync(&b, c, ns, na, ni, st, stream, fl);
        if (rc) return rc;
        if (!fl[TODE_FLAG_NEEDS_GENERAL]) {
            *iterations = fl[TODE_FLAG_MAX_ITERATIONS];
            return TODE_OK;
        }
        if (!small_system) return fail(TODE_E_UNSUPPORTED, "this batch leaves the case the whole-solve kernel of this term is built for");
    }

    // The general kernel: every case.  Up to three launches, each followed by a look at its flag words.
    b.flags = (int32_t *)(ws + w.flags);
    int32_t *counters = (int32_t *)(ws + w.counters);
    b.n_steps = counters, b.n_accepted = counters + B, b.n_initialized = counters + 2 * B, b.status_last = counters + 3 * B, b.status_idle = counters + 4 * B;
    int32_t fl[TODE_FLAG_WORDS] = {0, INT_MAX, 0, 0};
    auto run = [&]() -> int {
        int rc = tode_solve_builtin(&b, c, stream);
        if (rc) return rc;
        rc = check_hip(hipMemcpyAsync(fl, b.flags, sizeof(fl), hipMemcpyDeviceToHost, s), "tode_solve_builtin_auto: reading the flag words");
        if (rc) return rc;
        return check_hip(hipStreamSynchronize(s), "tode_solve_builtin_auto: waiting for the solve");
    };
    int rc = run();
    if (rc) return rc;
    if (fl[TODE_FLAG_NON_MONOTONE]) {  // some row of evaluation points is not monotone in its direction of time: again, with a mask
        b.pending = ws + w.pending;
        if ((rc = run())) return rc;
    }
    const int64_t most = fl[TODE_FLAG_MAX_ITERATIONS], first_failure = fl[TODE_FLAG_FIRST_FAILURE];
    const int64_t last = most < first_failure ? most : first_failure;
    if (last < most) {  // a non-success status stops the whole batch at iteration `last` (adjoints.py:229-238)
        b.iteration_cap = last;
        if ((rc = run())) return rc;
    }
    *iterations = last;
    return tode_finalize_stats(B, last, b.n_steps, b.n_accepted, b.n_initialized, b.status_last, b.status_idle, ns, na, ni, st, data_type(a->dtype), a->n_features,
                               a->n_eval, a->ys, b.y_idle, stream);
}

}  // extern "C"
