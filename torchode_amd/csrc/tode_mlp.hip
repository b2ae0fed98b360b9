// Whole-solve kernel for a two-layer perceptron right-hand side shared by the batch,
//   f(t, y) = tanh([y, t] W1^T + b1) W2^T + b2,   y in R^64, 256 hidden units, float32,
// with both matrix products on the matrix cores (v_mfma_f32_16x16x4_f32).
//
// One workgroup of four wavefronts advances a tile of 16 samples.  Both layers are computed
// transposed, weights as the A operand (rows) and samples as columns, so that
//   * the weights never move after the prologue: every lane keeps, in registers, exactly the
//     A operands its wavefront feeds to the matrix cores -- wavefront w owns hidden units
//     64w..64w+63: their rows of W1 (17 k-steps x 4 tiles = 68 registers) and their columns
//     of W2 (4 output tiles x 16 k-steps = 64 registers);
//   * layer 1, H^T = W1 [y, t]^T: the stage input [16 x 65] goes to LDS once, every wavefront
//     reads it as the B operand; the result tile, lane (q = lane/16, c = lane%16) holding hidden
//     units 4q..4q+3 of sample c, is -- after tanh -- already laid out as the B operand of
//     layer 2 for k-steps over exactly those hidden units.  No trip through LDS between the layers;
//   * layer 2: every wavefront multiplies its 64 hidden units into partial sums of all 64
//     outputs; the four partial sums meet in LDS (one 16-byte write and read per lane and tile).
//     Two barriers per evaluation of f;
//   * the result layout is the layout of the solver state: lane (q, c) of wavefront w holds
//     features 16w + 4q .. 16w + 4q + 3 of sample c, for y, the seven stage derivatives and the
//     dense-output coefficients (16-byte accesses to y0 and ys).  Per-sample scalars (t, dt,
//     error ratio, counters) are carried redundantly by the 16 lanes that share a sample.
//
// The weights are read in a packed order (tode_mlp_pack_weights): registers 4i..4i+3 of thread
// tid as one 16-byte value at packed[(i * 256 + tid) * 4], so that the prologue is 38 loads per
// thread, each contiguous across a wavefront.
//
// Same contract as the other fast kernels: the common case only; anything else raises
// TODE_FLAG_NEEDS_GENERAL and leaves the outputs unspecified.
#include <limits.h>

#include "tode_solve.h"

namespace tode {

typedef float mfma_acc __attribute__((ext_vector_type(4)));

struct MlpOut {
    int64_t *n_steps, *n_accepted, *n_initialized, *status;
    int n_features;  // features of the problem: at most 64 (the kernel's others stay zero)
};

constexpr int MLP_F = 64, MLP_H = 256, MLP_TILE = 16;
// LDS row of the stage input: 64 features, t, zeros up to column 79; padded to 100 values = 4 banks past a multiple of
// 32, so that the 16-byte reads and writes of eight lanes that differ in their sample fall on 32 different banks
constexpr int MLP_XS = 100;
constexpr int MLP_REGS = 68 + 16 + 64 + 4;       // packed values per thread: W1, b1, W2, b2
constexpr int MLP_REGS_BF16 = 40 + 16 + 32 + 4;  // the same with W1 (80 inputs) and W2 as pairs of bfloat16

struct __align__(16) MlpShared {
    float x[MLP_TILE * MLP_XS];
    float part[4][4][64][4];        // [output tile][wavefront it comes from][lane][4 features]
    float red[2][4][MLP_TILE][2];   // per-wavefront partial sums of up to two per-sample reductions
    int vote[2][4];                 // per-wavefront bits of the workgroup-wide "or"
};

struct MlpWeights {
    float w1[17][4];    // W1[64w + 16 tile + c][input of (kk, q)]
    float b1[4][4];     // b1[64w + 16 tile + 4q + r]
    float w2[4][4][4];  // W2[16 ft + c][64w + 16 tile + 4q + r]
    float b2[4];        // b2[16w + 4q + r]
};

// The variant with bfloat16 inputs to the matrix cores (v_mfma_f32_16x16x16_bf16: 16 k per
// instruction, a lane supplies k = 4q..4q+3): float32 accumulation, biases, tanh and solver state.
typedef __bf16 mlp_bf16x4 __attribute__((ext_vector_type(4)));
typedef unsigned mlp_u32x2 __attribute__((ext_vector_type(2)));

struct MlpWeightsBf16 {
    mlp_bf16x4 w1[5][4];  // W1[64w + 16 tile + c][16 ks + 4q + j], inputs 65..79 are zero
    float b1[4][4];
    mlp_bf16x4 w2[4][4];  // [ft][tile]: W2[16 ft + c][64w + 16 tile + 4q + j]
    float b2[4];
};

// Which input column lane group q feeds at k-step kk of the first layer: 16 features each for
// the first 16 steps (contiguous in LDS), then t and three zero columns.
__host__ __device__ __forceinline__ int mlp_input_of(int kk, int q) { return kk < 16 ? 16 * q + kk : 64 + q; }

// Source index (in W1 | b1 | W2 | b2, row-major) of packed value j of thread tid, or -1 for zero.  H: hidden units of
// the network at hand, at most MLP_H; the kernel's units from H on get zero weights and a zero bias, so that they
// add tanh(0) * 0 = 0 to every sum in the same places as before (a narrower network in the same arithmetic).
// FR: features of the network at hand (at most MLP_F): W1 is [H x (FR + 1)] with the time in its last
// column, W2 [FR x H]; the kernel's features from FR on get zero weights on both sides and stay zero throughout.
__host__ __device__ inline long long mlp_packed_source(int j, int tid, int H, int FR) {
    const int lane = tid & 63, w = tid >> 6, q = lane >> 4, c = lane & 15;
    const long long o_b1 = (long long)H * (FR + 1), o_w2 = o_b1 + H, o_b2 = o_w2 + (long long)FR * H;
    // column of W1 for the kernel's input k (features 0..63, then the time at 64), or -1
    auto w1_column = [&](int k) { return k < FR ? k : (k == MLP_F ? FR : -1); };
    if (j < 68) {
        const int kk = j / 4, tile = j % 4, col = w1_column(mlp_input_of(kk, q)), unit = 64 * w + 16 * tile + c;
        return (col >= 0 && unit < H) ? (long long)unit * (FR + 1) + col : -1;
    }
    j -= 68;
    if (j < 16) {
        const int unit = 64 * w + 16 * (j / 4) + 4 * q + (j % 4);
        return unit < H ? o_b1 + unit : -1;
    }
    j -= 16;
    if (j < 64) {
        const int ft = j / 16, tile = (j / 4) % 4, r = j % 4, unit = 64 * w + 16 * tile + 4 * q + r;
        return (unit < H && 16 * ft + c < FR) ? o_w2 + (long long)(16 * ft + c) * H + unit : -1;
    }
    j -= 64;
    return 16 * w + 4 * q + j < FR ? o_b2 + 16 * w + 4 * q + j : -1;
}

// The same for the bfloat16 variant: packed word j of thread tid holds the values of sources
// (lo, hi) as bfloat16 in its low and high half (words of b1 and b2: one float32, hi = -2).
__host__ __device__ inline void mlp_packed_source_bf16(int j, int tid, int H, int FR, long long &lo, long long &hi) {
    const int lane = tid & 63, w = tid >> 6, q = lane >> 4, c = lane & 15;
    const long long o_b1 = (long long)H * (FR + 1), o_w2 = o_b1 + H, o_b2 = o_w2 + (long long)FR * H;
    auto w1_column = [&](int k) { return k < FR ? k : (k == MLP_F ? FR : -1); };
    hi = -2;
    if (j < 40) {
        const int ks = j / 8, tile = (j / 2) % 4, k = 16 * ks + 4 * q + 2 * (j % 2), unit = 64 * w + 16 * tile + c;
        const long long row = (long long)unit * (FR + 1);
        lo = (w1_column(k) >= 0 && unit < H) ? row + w1_column(k) : -1;
        hi = (w1_column(k + 1) >= 0 && unit < H) ? row + w1_column(k + 1) : -1;
        return;
    }
    j -= 40;
    if (j < 16) {
        const int unit = 64 * w + 16 * (j / 4) + 4 * q + (j % 4);
        lo = unit < H ? o_b1 + unit : -1;
        hi = -3;  // (one float32 word, zero where lo < 0)
        return;
    }
    j -= 16;
    if (j < 32) {
        const int ft = j / 8, tile = (j / 2) % 4, unit = 64 * w + 16 * tile + 4 * q + 2 * (j % 2);
        const long long at = o_w2 + (long long)(16 * ft + c) * H + unit;
        lo = (unit < H && 16 * ft + c < FR) ? at : -1;
        hi = (unit + 1 < H && 16 * ft + c < FR) ? at + 1 : -1;
        return;
    }
    j -= 32;
    lo = 16 * w + 4 * q + j < FR ? o_b2 + 16 * w + 4 * q + j : -1;
}

static __global__ void mlp_pack_bf16_kernel(const float *raw, unsigned *packed, int H, int FR) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= MLP_REGS_BF16 * 256) return;
    const int part = i % 4, tid = (i / 4) % 256, group = i / 1024;
    long long lo, hi;
    mlp_packed_source_bf16(4 * group + part, tid, H, FR, lo, hi);
    if (hi == -2 || hi == -3) {
        packed[i] = lo < 0 ? 0u : __float_as_uint(raw[lo]);
        return;
    }
    const __bf16 a = (__bf16)(lo < 0 ? 0.0f : raw[lo]), b = (__bf16)(hi < 0 ? 0.0f : raw[hi]);  // round to nearest even
    packed[i] = (unsigned)__builtin_bit_cast(unsigned short, a) | ((unsigned)__builtin_bit_cast(unsigned short, b) << 16);
}

static __global__ void mlp_pack_kernel(const float *raw, float *packed, int H, int FR) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= MLP_REGS * 256) return;
    const int part = i % 4, tid = (i / 4) % 256, group = i / 1024;
    const long long src = mlp_packed_source(4 * group + part, tid, H, FR);
    packed[i] = src < 0 ? 0.0f : raw[src];
}

// Bitwise "or" of `bits` over the workgroup (four wavefronts).  Consecutive calls alternate between
// two sets of LDS words, so a wavefront that runs ahead into the next call cannot overwrite what
// a slower one still has to read.
__device__ __forceinline__ int block_or(MlpShared &sh, int &vslot, int bits) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) bits |= __shfl_xor(bits, off);
    if (lane == 0) sh.vote[vslot][w] = bits;
    lds_barrier();
    const int all = (sh.vote[vslot][0] | sh.vote[vslot][1]) | (sh.vote[vslot][2] | sh.vote[vslot][3]);
    vslot ^= 1;
    return all;
}

// tanh(x) = 1 - 2 / (exp(2x) + 1) on the hardware exp2 and reciprocal: absolute error about 2e-7
// (the library tanhf costs several times the matrix products of a layer).  exp2 overflows to inf
// and underflows to 0 exactly where tanh saturates, so no range checks are needed.
__device__ __forceinline__ float mlp_tanh(float x) {
    const float e = __builtin_amdgcn_exp2f(x * 2.8853900817779268f);  // 2 / ln 2
    return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
}

// out[r] = f(tn, yi)[16w + 4q + r] for the lane's sample.
__device__ __forceinline__ void mlp_rhs(MlpShared &sh, const MlpWeights &W, float tn, const float (&yi)[4], float (&out)[4]) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, q = lane >> 4, c = lane & 15;
    *reinterpret_cast<float4 *>(sh.x + c * MLP_XS + 16 * w + 4 * q) = make_float4(yi[0], yi[1], yi[2], yi[3]);
    if (w == 0 && q == 0) sh.x[c * MLP_XS + MLP_F] = tn;
    lds_barrier();
    // all B operands of the layer into registers first, so that the matrix cores never wait for LDS
    float a1[17];
    {
        const float4 *row = reinterpret_cast<const float4 *>(sh.x + c * MLP_XS + 16 * q);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float4 v = row[j];
            a1[4 * j] = v.x, a1[4 * j + 1] = v.y, a1[4 * j + 2] = v.z, a1[4 * j + 3] = v.w;
        }
        a1[16] = sh.x[c * MLP_XS + MLP_F + q];
    }
    asm volatile("" ::: "memory");
    mfma_acc h[4];
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) h[tile] = {W.b1[tile][0], W.b1[tile][1], W.b1[tile][2], W.b1[tile][3]};
#pragma unroll
    for (int kk = 0; kk < 17; ++kk) {
#pragma unroll
        for (int tile = 0; tile < 4; ++tile) h[tile] = __builtin_amdgcn_mfma_f32_16x16x4f32(W.w1[kk][tile], a1[kk], h[tile], 0, 0, 0);
    }
#pragma unroll
    for (int tile = 0; tile < 4; ++tile)
#pragma unroll
        for (int r = 0; r < 4; ++r) h[tile][r] = mlp_tanh(h[tile][r]);
    mfma_acc acc[4];
#pragma unroll
    for (int ft = 0; ft < 4; ++ft) acc[ft] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int tile = 0; tile < 4; ++tile)
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int ft = 0; ft < 4; ++ft) acc[ft] = __builtin_amdgcn_mfma_f32_16x16x4f32(W.w2[ft][tile][r], h[tile][r], acc[ft], 0, 0, 0);
#pragma unroll
    for (int ft = 0; ft < 4; ++ft) *reinterpret_cast<float4 *>(sh.part[ft][w][lane]) = make_float4(acc[ft][0], acc[ft][1], acc[ft][2], acc[ft][3]);
    lds_barrier();
    float4 s[4];
#pragma unroll
    for (int from = 0; from < 4; ++from) s[from] = *reinterpret_cast<const float4 *>(sh.part[w][from][lane]);
    out[0] = ((s[0].x + s[1].x) + (s[2].x + s[3].x)) + W.b2[0];
    out[1] = ((s[0].y + s[1].y) + (s[2].y + s[3].y)) + W.b2[1];
    out[2] = ((s[0].z + s[1].z) + (s[2].z + s[3].z)) + W.b2[2];
    out[3] = ((s[0].w + s[1].w) + (s[2].w + s[3].w)) + W.b2[3];
}

__device__ __forceinline__ void mlp_rhs(MlpShared &sh, const MlpWeightsBf16 &W, float tn, const float (&yi)[4], float (&out)[4]) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, q = lane >> 4, c = lane & 15;
    *reinterpret_cast<float4 *>(sh.x + c * MLP_XS + 16 * w + 4 * q) = make_float4(yi[0], yi[1], yi[2], yi[3]);
    if (w == 0 && q == 0) sh.x[c * MLP_XS + MLP_F] = tn;
    lds_barrier();
    mlp_bf16x4 a1[5];
    {
        const float *row = sh.x + c * MLP_XS + 4 * q;
#pragma unroll
        for (int ks = 0; ks < 5; ++ks) {
            const float4 v = *reinterpret_cast<const float4 *>(row + 16 * ks);
            a1[ks] = {(__bf16)v.x, (__bf16)v.y, (__bf16)v.z, (__bf16)v.w};
        }
    }
    asm volatile("" ::: "memory");
    mfma_acc h[4];
#pragma unroll
    for (int tile = 0; tile < 4; ++tile) h[tile] = {W.b1[tile][0], W.b1[tile][1], W.b1[tile][2], W.b1[tile][3]};
#pragma unroll
    for (int ks = 0; ks < 5; ++ks) {
#pragma unroll
        for (int tile = 0; tile < 4; ++tile) h[tile] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(W.w1[ks][tile], a1[ks], h[tile], 0, 0, 0);
    }
    mlp_bf16x4 hb[4];
#pragma unroll
    for (int tile = 0; tile < 4; ++tile)
        hb[tile] = {(__bf16)mlp_tanh(h[tile][0]), (__bf16)mlp_tanh(h[tile][1]), (__bf16)mlp_tanh(h[tile][2]), (__bf16)mlp_tanh(h[tile][3])};
    mfma_acc acc[4];
#pragma unroll
    for (int ft = 0; ft < 4; ++ft) acc[ft] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int tile = 0; tile < 4; ++tile)
#pragma unroll
        for (int ft = 0; ft < 4; ++ft) acc[ft] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(W.w2[ft][tile], hb[tile], acc[ft], 0, 0, 0);
#pragma unroll
    for (int ft = 0; ft < 4; ++ft) *reinterpret_cast<float4 *>(sh.part[ft][w][lane]) = make_float4(acc[ft][0], acc[ft][1], acc[ft][2], acc[ft][3]);
    lds_barrier();
    float4 s[4];
#pragma unroll
    for (int from = 0; from < 4; ++from) s[from] = *reinterpret_cast<const float4 *>(sh.part[w][from][lane]);
    out[0] = ((s[0].x + s[1].x) + (s[2].x + s[3].x)) + W.b2[0];
    out[1] = ((s[0].y + s[1].y) + (s[2].y + s[3].y)) + W.b2[1];
    out[2] = ((s[0].z + s[1].z) + (s[2].z + s[3].z)) + W.b2[2];
    out[3] = ((s[0].w + s[1].w) + (s[2].w + s[3].w)) + W.b2[3];
}

// Packed weights (tode_mlp_pack_weights) into the registers of thread tid.
__device__ __forceinline__ void mlp_load(MlpWeights &W, const float *packed, int tid) {
    const float4 *src = reinterpret_cast<const float4 *>(packed) + tid;
    float v[MLP_REGS];
#pragma unroll
    for (int i = 0; i < MLP_REGS / 4; ++i) {
        const float4 u = src[i * 256];
        v[4 * i] = u.x, v[4 * i + 1] = u.y, v[4 * i + 2] = u.z, v[4 * i + 3] = u.w;
    }
#pragma unroll
    for (int j = 0; j < 68; ++j) W.w1[j / 4][j % 4] = v[j];
#pragma unroll
    for (int j = 0; j < 16; ++j) W.b1[j / 4][j % 4] = v[68 + j];
#pragma unroll
    for (int j = 0; j < 64; ++j) W.w2[j / 16][(j / 4) % 4][j % 4] = v[84 + j];
#pragma unroll
    for (int j = 0; j < 4; ++j) W.b2[j] = v[148 + j];
}

__device__ __forceinline__ void mlp_load(MlpWeightsBf16 &W, const float *packed, int tid) {
    const uint4 *src = reinterpret_cast<const uint4 *>(packed) + tid;
    unsigned v[MLP_REGS_BF16];
#pragma unroll
    for (int i = 0; i < MLP_REGS_BF16 / 4; ++i) {
        const uint4 u = src[i * 256];
        v[4 * i] = u.x, v[4 * i + 1] = u.y, v[4 * i + 2] = u.z, v[4 * i + 3] = u.w;
    }
#pragma unroll
    for (int j = 0; j < 20; ++j) W.w1[j / 4][j % 4] = __builtin_bit_cast(mlp_bf16x4, (mlp_u32x2){v[2 * j], v[2 * j + 1]});
#pragma unroll
    for (int j = 0; j < 16; ++j) W.b1[j / 4][j % 4] = __uint_as_float(v[40 + j]);
#pragma unroll
    for (int j = 0; j < 16; ++j) W.w2[j / 4][j % 4] = __builtin_bit_cast(mlp_bf16x4, (mlp_u32x2){v[56 + 2 * j], v[56 + 2 * j + 1]});
#pragma unroll
    for (int j = 0; j < 4; ++j) W.b2[j] = __uint_as_float(v[88 + j]);
}

// Per-sample sums over the 64 features of two quantities at once: the lane's four features, the
// four lane groups of a wavefront by shuffles, the four wavefronts through LDS.
__device__ __forceinline__ void mlp_sum2(MlpShared &sh, int &slot, const float (&a)[4], const float (&b)[4], float &A, float &B) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, q = lane >> 4, c = lane & 15;
    float u = (a[0] + a[1]) + (a[2] + a[3]), v = (b[0] + b[1]) + (b[2] + b[3]);
#pragma unroll
    for (int off = 16; off < 64; off <<= 1) {
        u = u + __shfl_xor(u, off);
        v = v + __shfl_xor(v, off);
    }
    if (q == 0) {
        sh.red[slot][w][c][0] = u;
        sh.red[slot][w][c][1] = v;
    }
    lds_barrier();
    A = (sh.red[slot][0][c][0] + sh.red[slot][1][c][0]) + (sh.red[slot][2][c][0] + sh.red[slot][3][c][0]);
    B = (sh.red[slot][0][c][1] + sh.red[slot][1][c][1]) + (sh.red[slot][2][c][1] + sh.red[slot][3][c][1]);
    slot ^= 1;
}

// FULL: all 64 state values are the problem's and evaluation points are given (the feature count and the end-point mode are
// constants and their tests fold away).
template <int METHOD, int CTRL, typename Weights, bool FULL>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) solve_mlp_kernel(const SolveParams<float> p, const float *packed, const MlpOut o) {
    using T = float;
    using Tab = typename std::conditional<METHOD == 1, Tsit5Tab, Dopri5Tab>::type;
    constexpr int F = MLP_F;
    __shared__ MlpShared sh;
    extern __shared__ __align__(16) unsigned char dyn[];
    T *te_s = reinterpret_cast<T *>(dyn);  // [16][E]

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, q = lane >> 4, c = lane & 15;
    const long long b0 = (long long)blockIdx.x * MLP_TILE;
    const int rows = (int)min((long long)MLP_TILE, p.batch - b0);
    // Without evaluation points (the end point alone, adjoints.py:296-311) t_end is every sample's one point: ys takes the
    // dense output of the sample's last step there and y_idle its final state; the caller picks per sample
    // (tode_select_end_point).
    const bool end_only = !FULL && p.n_eval == 0;
    const int E = end_only ? 1 : p.n_eval;
    const CtrlParams<T> &cp = p.cp;
    const int FR = FULL ? MLP_F : o.n_features;  // the problem's features; the kernel's others (FR .. 63) are zero in every vector
    const T sf = (T)__builtin_sqrt((double)FR);
    const int f0 = 16 * w + 4 * q;  // the lane's first feature
    const bool has = f0 < FR;       // (some of the lane's four features are the problem's)
    const bool quads = (FR & 3) == 0;  // rows of whole groups of four: 16-byte loads and stores
    auto put = [&](T *row, const T (&v)[4]) {  // the lane's share of one row of ys
        if (quads) {
            if (has) *reinterpret_cast<float4 *>(row + f0) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (f0 + r < FR) row[f0 + r] = v[r];
        }
    };
    int slot = 0;

    // ---- state of the lane's sample (asked for first: these loads are on their way while the weights arrive) ----
    const bool live = c < rows;
    const long long bs = b0 + (live ? c : 0);
    const T ts = p.t_start[bs * p.ts_stride], te = p.t_end[bs * p.te_stride];
    T y[4], k[7][4];
    {
        if (quads) {
            const float4 v = has ? *reinterpret_cast<const float4 *>(p.y0 + bs * FR + f0) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            y[0] = v.x, y[1] = v.y, y[2] = v.z, y[3] = v.w;
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) y[r] = f0 + r < FR ? p.y0[bs * FR + f0 + r] : 0.0f;
        }
    }

    // ---- weights into registers ----
    Weights W;
    mlp_load(W, packed, tid);
    for (int i = tid; i < MLP_TILE * MLP_XS; i += 256) sh.x[i] = 0.0f;  // also the zero columns from 65 on
    for (int i = tid; i < rows * E; i += 256) te_s[i] = end_only ? p.t_end[(b0 + i) * p.te_stride] : p.t_eval[b0 * E + i];
    __syncthreads();

    const T *tev = te_s + (live ? c : 0) * E;
    const T dir = (te > ts) ? (T)1 : (T)-1, tlo = tmin(ts, te), thi = tmax(te, ts);
    bool bail = false;
    // not monotone: the sixteen threads that share the sample (four lane groups in each of four wavefronts) split its
    // neighbouring pairs among them; the workgroup's vote below collects what any of them found
    for (int e = 1 + q + 4 * w; e < E; e += 16) bail = bail || (live && !(dir * tev[e] >= dir * tev[e - 1]));
    T t = ts, dt, prev = 1, pprev = 1;
    int cursor = 0, n_steps = 0, n_acc = 0;

    // ---- first step size (step_size_controllers.py:431-490, 776-835) ----
    mlp_rhs(sh, W, ts, y, k[0]);
    if (p.dt0) {
        dt = p.dt0[bs];
    } else {
        T inv[4], a0[4], a1[4], y1[4], f1[4], A0, A1, A2;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            inv[r] = inv_scale(cp.atol, cp.rtol, y[r]);
            const T x0 = (y[r] * inv[r]) / sf, x1 = (k[0][r] * inv[r]) / sf;
            a0[r] = x0 * x0;
            a1[r] = x1 * x1;
        }
        mlp_sum2(sh, slot, a0, a1, A0, A1);
        const T d0 = sqrt_(A0), d1 = sqrt_(A1);
        const T h = (d0 < (T)1e-5 || d1 < (T)1e-5) ? (T)1e-6 : ((T)0.01 * d0) / d1;
        const T h0 = tmin(h, abs_(te - ts));
#pragma unroll
        for (int r = 0; r < 4; ++r) y1[r] = fma_(dir * h0, k[0][r], y[r]);
        mlp_rhs(sh, W, fma_(dir, h0, ts), y1, f1);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const T x2 = ((f1[r] - k[0][r]) * inv[r]) / sf;
            a0[r] = x2 * x2;
        }
        mlp_sum2(sh, slot, a0, a1, A2, A1);  // A1 (the norm of f0) comes out again unchanged
        dt = initial_finish<T>(CTRL == 1 ? TODE_CTRL_PID : TODE_CTRL_INTEGRAL, 1.0 / 5.0, dir, h0, sqrt_(A1), sqrt_(A2));
    }
    dt = tclamp(dt, tlo - t, thi - t);
    bool active = live;
    if (live && E > 0 && tev[0] == ts) {
        put(p.ys + (bs * E) * FR, y);
        cursor = 1;
    }
    int vslot = 0;
    // bit 1: some sample needs the general kernel; bit 0: some sample still runs
    int state = block_or(sh, vslot, (bail ? 2 : 0) | (active ? 1 : 0));
    bail = (state & 2) != 0;
    // A sample that has landed past t_end (t + (t_end - t) rounded upwards) keeps stepping in the reference's later
    // iterations with the clamped step t_end - t, which is seen only in the status of that step: the sample sits
    // through one more iteration here, inactive, and the status of its step is looked at.
    bool idle = false, idle_done = false;
    while (state == 1) {
        // ---- stages (runge_kutta.py:255-263) ----
        const T t0 = t;
        T y1[4];
#pragma unroll
        for (int i = 1; i < 7; ++i) {
            T yi[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                T s = 0;
#pragma unroll
                for (int j = 0; j < i; ++j) s = fma_((T)Tab::a[i][j], k[j][r], s);
                yi[r] = fma_(dt, s, y[r]);
            }
            mlp_rhs(sh, W, fma_((T)Tab::c[i], dt, t0), yi, k[i]);
            if (i == 6) {
#pragma unroll
                for (int r = 0; r < 4; ++r) y1[r] = yi[r];
            }
        }

        // ---- error ratio (runge_kutta.py:267, step_size_controllers.py:389-395); F >= 58: fused sums ----
        T part[4], zero[4] = {0, 0, 0, 0}, total, unused;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            T err = 0;
#pragma unroll
            for (int s = 0; s < 7; ++s) err = fma_(dt * (T)Tab::b_err[s], k[s][r], err);
            const T m = tmax(abs_(y[r]), abs_(y1[r]));
            const T x = (abs_(err) / fma_(cp.rtol, m, cp.atol)) / sf;
            part[r] = x * x;
        }
        mlp_sum2(sh, slot, part, zero, total, unused);

        const T ratio = tmax(sqrt_(total), (T)1e-38);
        const bool accept = ratio < (T)1;
        T dt_next = dt * dt_factor<T, CTRL>(cp, ratio, prev, pprev);
        const int status = limit_dt<T>(cp, ratio, dt_next);
        bail = bail || (idle && status != 0);
        // (without evaluation points the end point of such a sample is this step's interpolant at t_end: below)
        const bool idle_point = idle && end_only;
        idle = false;
        const bool move = accept && active;
        const T t_new = move ? (t0 + dt) : t0;
        const bool running_new = fma_(dir, t_new, -dir * te) < (T)0;
        n_steps += active ? 1 : 0;
        n_acc += move ? 1 : 0;

        // ---- dense output at the evaluation points this step passed (adjoints.py:215-234) ----
        if (idle_point || (active && cursor < E && fma_(dir, t_new, -dir * tev[cursor]) >= (T)0)) {
            T qc[4][5][1];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                T ks[7];
#pragma unroll
                for (int s = 0; s < 7; ++s) ks[s] = k[s][r];
                // (one fused chain per coefficient, ATen's form for rows of 58 values and more; for a shorter row ATen rounds
                // the products first, a difference at the level of this kernel's matrix products against torch's)
                quartic_elem<T, METHOD>(dt, y[r], y1[r], ks, true, qc[r]);
            }
            const T t1 = t0 + dt;
            do {
                const T x = unit_time(idle_point ? te : tev[cursor], t0, t1);
                T v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    v[r] = qc[r][4][0];
#pragma unroll
                    for (int pw = 3; pw >= 0; --pw) v[r] = fma_(v[r], x, qc[r][pw][0]);
                }
                if (idle_point) {
                    put(p.y_idle + bs * FR, v);
                    idle_done = true;
                    break;
                }
                put(p.ys + (bs * E + cursor) * FR, v);
                ++cursor;
            } while (cursor < E && fma_(dir, t_new, -dir * tev[cursor]) >= (T)0);
        }

        // ---- state update (adjoints.py:150-155, 247-255) ----
        bool nonfinite = false;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            y[r] = move ? y1[r] : y[r];
            k[0][r] = move ? k[6][r] : k[0][r];
            nonfinite = nonfinite || !settles_(y[r], k[0][r]);
        }
        t = t_new;
        const T dtc = tclamp(running_new ? dt_next : dt, tlo - t_new, thi - t_new);
        dt = active ? dtc : dt;
        if (CTRL == 1 && active && running_new && accept) {
            pprev = prev;
            prev = ratio;
        }
        const bool failed = active && (status != 0 || n_steps >= p.max_steps || n_steps >= TODE_HARD_STEP_LIMIT);
        const bool finished = active && !failed && !running_new;
        // a sample that ends on a non-finite value shows up in later iterations of the reference loop: not the
        // common case; one that landed past t_end is looked at in the next iteration
        bail = bail || failed || (finished && nonfinite);
        idle = finished && !nonfinite && !(t == te);
        active = active && !failed && running_new;
        state = block_or(sh, vslot, (bail ? 2 : 0) | ((active || idle) ? 1 : 0));
        bail = (state & 2) != 0;
    }

    if (end_only && live && !idle_done) put(p.y_idle + bs * FR, y);  // the final state
    if (w == 0) {
        if (q == 0 && live) {
            o.n_steps[bs] = n_steps;
            o.n_accepted[bs] = n_acc;
            o.n_initialized[bs] = cursor;
            o.status[bs] = 0;
        }
        // one update of each flag word per workgroup: four thousand atomic operations on one address would queue up
        // behind each other at the end of a kernel whose workgroups all finish together
        int most = live ? n_steps : 0;
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) most = max(most, __shfl_xor(most, off));
        if (lane == 0) {
            if (most > 0) atomicMax(&p.flags[TODE_FLAG_MAX_ITERATIONS], most);
            if (bail) atomicMax(&p.flags[TODE_FLAG_NEEDS_GENERAL], 1);  // (agreed on by the workgroup's last vote)
        }
    }
    publish_flags(p);
}

template <int METHOD, int CTRL, typename Weights> static int launch_mlp(const tode_solve_args &a, const tode_controller &c, const MlpOut &o, hipStream_t stream) {
    SolveParams<float> p = make_params<float>(a, c);
    reset_flags(a.flags, stream);
    if (a.batch == 0) return check_hip(hipGetLastError(), "tode_solve_builtin_fast launch");
    const size_t lds = (size_t)MLP_TILE * (a.n_eval > 0 ? a.n_eval : 1) * sizeof(float);
    const unsigned blocks = (unsigned)((a.batch + MLP_TILE - 1) / MLP_TILE);
    timing_before(stream, std::is_same<Weights, MlpWeightsBf16>::value ? "tode::solve_mlp_kernel (bfloat16 matrix inputs)" : "tode::solve_mlp_kernel");
    if (o.n_features == MLP_F && a.n_eval > 0)
        hipLaunchKernelGGL((solve_mlp_kernel<METHOD, CTRL, Weights, true>), dim3(blocks), dim3(256), lds, stream, p, (const float *)a.shared_params, o);
    else
        hipLaunchKernelGGL((solve_mlp_kernel<METHOD, CTRL, Weights, false>), dim3(blocks), dim3(256), lds, stream, p, (const float *)a.shared_params, o);
    timing_after(stream);
    return check_hip(hipGetLastError(), "tode_solve_builtin_fast launch");
}

template <typename Weights> static int solve_mlp_with(const tode_solve_args &a, const tode_controller &c, const MlpOut &o, hipStream_t s) {
    if (a.method == TODE_DOPRI5 && c.kind == TODE_CTRL_INTEGRAL) return launch_mlp<0, 0, Weights>(a, c, o, s);
    if (a.method == TODE_DOPRI5 && c.kind == TODE_CTRL_PID) return launch_mlp<0, 1, Weights>(a, c, o, s);
    if (a.method == TODE_TSIT5 && c.kind == TODE_CTRL_INTEGRAL) return launch_mlp<1, 0, Weights>(a, c, o, s);
    if (a.method == TODE_TSIT5 && c.kind == TODE_CTRL_PID) return launch_mlp<1, 1, Weights>(a, c, o, s);
    return fail(TODE_E_INVALID, "unknown method %d or controller kind %d", a.method, c.kind);
}

int solve_mlp_f32(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s) {
    const bool f32 = a.n_shared_params == (long long)TODE_MLP_PACKED_SIZE, bf16 = a.n_shared_params == (long long)TODE_MLP_PACKED_SIZE_BF16;
    if (a.n_features < 1 || a.n_features > MLP_F || !(f32 || bf16))
        return fail(TODE_E_UNSUPPORTED,
                    "the MLP kernel is built for 1 to 64 features and up to 256 hidden units, with the weights packed by tode_mlp_pack_weights "
                    "(%d or %d values); got F=%d and %lld shared parameters", TODE_MLP_PACKED_SIZE, TODE_MLP_PACKED_SIZE_BF16, a.n_features,
                    (long long)a.n_shared_params);
    if (!a.shared_params) return fail(TODE_E_INVALID, "null shared_params");
    if (a.n_eval > 512) return fail(TODE_E_UNSUPPORTED, "n_eval=%d is too large for the MLP kernel", a.n_eval);
    if (a.batch > (long long)INT_MAX * MLP_TILE) return fail(TODE_E_UNSUPPORTED, "batch too large");
    MlpOut o{ns, na, ni, st, a.n_features};
    return f32 ? solve_mlp_with<MlpWeights>(a, c, o, s) : solve_mlp_with<MlpWeightsBf16>(a, c, o, s);
}

int mlp_pack_weights(const float *raw, long long n_raw, int n_features, int matrix_inputs, float *packed, hipStream_t s) {
    static_assert(TODE_MLP_PACKED_SIZE == MLP_REGS * 256 && TODE_MLP_PACKED_SIZE_BF16 == MLP_REGS_BF16 * 256, "packed sizes");
    if (!raw || !packed) return fail(TODE_E_INVALID, "null pointer");
    const long long FR = n_features;
    if (FR < 1 || FR > MLP_F) return fail(TODE_E_UNSUPPORTED, "the MLP kernel takes 1 to %d features, got %lld", MLP_F, FR);
    // W1 [H x (F + 1)] | b1 [H] | W2 [F x H] | b2 [F] = (2 F + 2) H + F values for H hidden units, 1 <= H <= 256
    const long long H = (n_raw - FR) / (2 * FR + 2);
    if (n_raw < FR || H * (2 * FR + 2) + FR != n_raw || H < 1 || H > MLP_H)
        return fail(TODE_E_UNSUPPORTED, "expected W1 [H x %lld] | b1 [H] | W2 [%lld x H] | b2 [%lld] = %lld H + %lld values with 1 <= H <= %d, got %lld", FR + 1, FR, FR,
                    2 * FR + 2, FR, MLP_H, n_raw);
    if (matrix_inputs == TODE_MLP_INPUTS_F32)
        hipLaunchKernelGGL(mlp_pack_kernel, dim3((MLP_REGS * 256 + 255) / 256), dim3(256), 0, s, raw, packed, (int)H, (int)FR);
    else if (matrix_inputs == TODE_MLP_INPUTS_BF16)
        hipLaunchKernelGGL(mlp_pack_bf16_kernel, dim3((MLP_REGS_BF16 * 256 + 255) / 256), dim3(256), 0, s, raw, reinterpret_cast<unsigned *>(packed), (int)H, (int)FR);
    else
        return fail(TODE_E_INVALID, "unknown matrix input type %d", matrix_inputs);
    return check_hip(hipGetLastError(), "tode_mlp_pack_weights launch");
}

}  // namespace tode
