// Measurement aid: how often one SIMD of this GPU issues a vector instruction of a wavefront, as a function of
// how many wavefronts share the SIMD and how many independent dependency chains each of them runs.  The whole-solve
// kernels for the small systems are bound by exactly that (one sample per lane, a few hundred dependent vector
// instructions per Runge-Kutta step, one or two wavefronts per SIMD at the batch sizes they are used for), so this
// is the rate their per-step cost is to be read against.  No counterpart in the reference.
#include <vector>

#include "tode_internal.h"
#include "tode_math.h"

namespace tode {

constexpr int PROBE_INSTRUCTIONS = 16384;  // vector instructions per wavefront between the two readings of the clock

// OP 0: fused multiply-add; 1: correctly rounded division; 2: correctly rounded square root (each followed by the
// addition that keeps its argument in range: counted as one operation).
template <typename T, int CHAINS, int OP> __global__ void __launch_bounds__(64) probe_kernel(long long *ticks, T *sink, T a, T b) {
    T x[CHAINS];
#pragma unroll
    for (int c = 0; c < CHAINS; ++c) x[c] = (T)threadIdx.x * (T)1e-3 + (T)c;
    constexpr int per_chain = PROBE_INSTRUCTIONS / CHAINS / (OP == 0 ? 1 : 8);
    constexpr int UNROLL = (OP == 0 ? 64 : 8) / CHAINS;  // (loop bodies of 64 multiply-adds, or 8 of the long operations)
    const long long t0 = wall_clock64();  // (the constant 100 MHz counter: the shader clock itself varies with load)
#pragma unroll UNROLL
    for (int i = 0; i < per_chain; ++i) {
#pragma unroll
        for (int c = 0; c < CHAINS; ++c) {
            if (OP == 0) x[c] = fma_(x[c], a, b);
            if (OP == 1) x[c] = a / (x[c] + b);
            if (OP == 2) x[c] = sqrt_(x[c] + b);
        }
    }
    const long long t1 = wall_clock64();
    T sum = 0;
#pragma unroll
    for (int c = 0; c < CHAINS; ++c) sum += x[c];
    sink[(long long)blockIdx.x * 64 + threadIdx.x] = sum;  // (keeps the chains alive)
    if (threadIdx.x == 0) ticks[2 * blockIdx.x] = t0, ticks[2 * blockIdx.x + 1] = t1;
}

template <typename T, int OP> static int probe_chains(int chains, unsigned blocks, long long *ticks, T *sink, hipStream_t s) {
    const T a = (T)1.0001, b = (T)0.5;
    switch (chains) {
    case 1: hipLaunchKernelGGL((probe_kernel<T, 1, OP>), dim3(blocks), dim3(64), 0, s, ticks, sink, a, b); break;
    case 2: hipLaunchKernelGGL((probe_kernel<T, 2, OP>), dim3(blocks), dim3(64), 0, s, ticks, sink, a, b); break;
    case 4: hipLaunchKernelGGL((probe_kernel<T, 4, OP>), dim3(blocks), dim3(64), 0, s, ticks, sink, a, b); break;
    case 8: hipLaunchKernelGGL((probe_kernel<T, 8, OP>), dim3(blocks), dim3(64), 0, s, ticks, sink, a, b); break;
    default: return fail(TODE_E_INVALID, "chains must be 1, 2, 4 or 8, got %d", chains);
    }
    return check_hip(hipGetLastError(), "tode_probe_vector_issue launch");
}

template <typename T> static int probe_op(int op, int chains, unsigned blocks, long long *ticks, void *sink, hipStream_t s) {
    if (op == 0) return probe_chains<T, 0>(chains, blocks, ticks, (T *)sink, s);
    if (op == 1) return probe_chains<T, 1>(chains, blocks, ticks, (T *)sink, s);
    if (op == 2) return probe_chains<T, 2>(chains, blocks, ticks, (T *)sink, s);
    return fail(TODE_E_INVALID, "unknown operation %d", op);
}

}  // namespace tode

extern "C" {

int64_t tode_probe_scratch_bytes(int32_t wavefronts) { return wavefronts < 1 ? -1 : (int64_t)wavefronts * (16 + 64 * 8); }

int tode_probe_vector_issue(int32_t dtype, int32_t operation, int32_t chains, int32_t wavefronts, void *scratch, int64_t scratch_bytes,
                            double *ns_per_operation, void *stream) {
    using namespace tode;
    if (!scratch || !ns_per_operation) return fail(TODE_E_INVALID, "null pointer");
    if (dtype != TODE_F32 && dtype != TODE_F64) return fail(TODE_E_INVALID, "dtype must be TODE_F32 or TODE_F64");
    if (wavefronts < 1 || wavefronts > (1 << 20)) return fail(TODE_E_INVALID, "wavefronts out of range: %d", wavefronts);
    if (scratch_bytes < tode_probe_scratch_bytes(wavefronts))
        return fail(TODE_E_INVALID, "the scratch buffer holds %lld bytes, the probe needs %lld (tode_probe_scratch_bytes)", (long long)scratch_bytes,
                    (long long)tode_probe_scratch_bytes(wavefronts));
    hipStream_t s = (hipStream_t)stream;
    long long *ticks = (long long *)scratch;
    void *sink = (void *)(ticks + 2 * (size_t)wavefronts);
    int rc = TODE_OK;
    for (int round = 0; round < 2 && rc == TODE_OK; ++round)  // (the first launch warms the instruction cache)
        rc = dtype == TODE_F32 ? probe_op<float>(operation, chains, (unsigned)wavefronts, ticks, sink, s)
                               : probe_op<double>(operation, chains, (unsigned)wavefronts, ticks, sink, s);
    if (rc) return rc;
    std::vector<long long> host(2 * (size_t)wavefronts);
    rc = check_hip(hipMemcpyAsync(host.data(), ticks, host.size() * 8, hipMemcpyDeviceToHost, s), "tode_probe_vector_issue: reading the tick counts");
    if (rc) return rc;
    rc = check_hip(hipStreamSynchronize(s), "tode_probe_vector_issue: waiting for the probe");
    if (rc) return rc;
    // The counter is one for the whole GPU.  From the first wavefront's start to the last one's end every SIMD has
    // issued its share of the wavefronts' operations, whatever order it took them in; how long one wavefront was at
    // it says less (a SIMD serves its oldest wavefront first).
    long long first = host[0], last = host[1];
    for (size_t w = 0; w < (size_t)wavefronts; ++w) first = host[2 * w] < first ? host[2 * w] : first, last = host[2 * w + 1] > last ? host[2 * w + 1] : last;
    const int operations = PROBE_INSTRUCTIONS / chains / (operation == 0 ? 1 : 8) * chains;
    *ns_per_operation = (double)(last - first) * 10.0 / operations;  // (10 ns per tick)
    return TODE_OK;
}

}  // extern "C"
