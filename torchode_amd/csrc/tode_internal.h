// Host-side helpers shared by the translation units of libtorchode_amd.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/torchode_amd.h"

// No sample may take more than this many steps.  The reference has no such limit (without
// max_steps a step size that has underflowed to zero makes its loop spin forever); a kernel
// that never ends would take the whole GPU with it, so the loop is cut here: the fast kernels
// hand the batch to the general one, which reports TODE_GENERAL_ERROR for the sample.
#ifndef TODE_HARD_STEP_LIMIT
#define TODE_HARD_STEP_LIMIT (1 << 22)
#endif

#define TODE_BLOCK 64  // one wavefront per workgroup: B/64 workgroups spread over all CUs and XCDs

#ifndef TODE_INSTANTIATE_F32
#define TODE_INSTANTIATE_F32 0
#endif
#ifndef TODE_INSTANTIATE_F64
#define TODE_INSTANTIATE_F64 0
#endif
#ifndef TODE_INSTANTIATE_T64_Y32
#define TODE_INSTANTIATE_T64_Y32 0
#endif
#ifndef TODE_INSTANTIATE_T32_Y64
#define TODE_INSTANTIATE_T32_Y64 0
#endif
#ifndef TODE_INSTANTIATE_RECORD
#define TODE_INSTANTIATE_RECORD 0
#endif

namespace tode {
// The two halves of a dtype argument: a plain TODE_F32 / TODE_F64 means both, TODE_DTYPES(data, time) names each.
inline int data_type(int32_t dtype) { return (dtype & TODE_DTYPE_PAIR) ? (dtype & 0xF) : dtype; }
inline int time_type(int32_t dtype) { return (dtype & TODE_DTYPE_PAIR) ? ((dtype >> 4) & 0xF) : dtype; }
inline bool known_dtype(int32_t dtype) {
    const int d = data_type(dtype), t = time_type(dtype);
    return (d == TODE_F32 || d == TODE_F64) && (t == TODE_F32 || t == TODE_F64) && !(dtype & ~(TODE_DTYPE_PAIR | 0xFF));
}

// Records a formatted message for tode_last_error() and returns `code`.
int fail(int code, const char *fmt, ...);
// Maps a HIP error to TODE_E_HIP (recording its string) or returns TODE_OK.
int check_hip(hipError_t err, const char *what);

// Set on the calling thread while tode_solve_builtin_fast_sync runs: the solve kernel then works on
// the library's own, self-resetting flag words `dev` (no reset launch in front of it) and its last
// workgroup stores the result, followed by `sequence`, into the pinned host words `host`.
// tode_solve_builtin_fast_static sets it too: `dev` are words of the library's static device array,
// `host` is the caller's flag block in device memory, and `sequence` is 0 (no word is written
// behind the flags; the caller reads them in stream order).
struct FlagTarget {
    int32_t *dev;
    int32_t *host;
    int32_t sequence;
};
const FlagTarget *flag_target();


// Event pair around the solve kernel, active only while timing is enabled on this thread.
void timing_before(hipStream_t s, const char *kernel_name);
void timing_after(hipStream_t s);

int solve_builtin_f32(const tode_solve_args &a, const tode_controller &c, hipStream_t s);
int solve_builtin_f64(const tode_solve_args &a, const tode_controller &c, hipStream_t s);
int solve_builtin_t64_y32(const tode_solve_args &a, const tode_controller &c, hipStream_t s);
int solve_builtin_t32_y64(const tode_solve_args &a, const tode_controller &c, hipStream_t s);
int solve_builtin_f32_record(const tode_solve_args &a, const tode_controller &c, hipStream_t s);
int solve_builtin_f64_record(const tode_solve_args &a, const tode_controller &c, hipStream_t s);
int solve_builtin_t64_y32_record(const tode_solve_args &a, const tode_controller &c, hipStream_t s);
int solve_builtin_t32_y64_record(const tode_solve_args &a, const tode_controller &c, hipStream_t s);
int solve_fast_f32(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s);
int solve_pair_f32(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s, bool *used);
int solve_pair_f64(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s, bool *used);
int solve_pair_f32_record(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s, bool *used);
int solve_pair_f64_record(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s, bool *used);
int solve_mlp_f32(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s);
int mlp_pack_weights(const float *raw, long long n_raw, int n_features, int matrix_inputs, float *packed, hipStream_t s);
int solve_grid_f32(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s);
int solve_grid_f64(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s);
int solve_fast_f64(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s);
int solve_fast_f32_record(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s);
int solve_fast_f64_record(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s);
}  // namespace tode
