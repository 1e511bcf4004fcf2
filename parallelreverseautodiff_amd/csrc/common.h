// Shared declarations of the prad_hip library internals (not part of the public ABI).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// The reference's runtime rounds every multiply and add separately (no fused multiply-add), so
// the elementwise arithmetic of this library is compiled without contraction as well.
#pragma clang fp contract(off)

namespace prad {

// Activation selectors: same values as PRAD_ACT_* in include/prad_hip.h.
enum Act : int { ACT_NONE = 0, ACT_LEAKYRELU = 1, ACT_SIGMOID = 2, ACT_TANH = 3, ACT_GELU = 4, ACT_AMPLIFIED_SIGMOID = 5 };
constexpr int ACT_LAST = ACT_AMPLIFIED_SIGMOID;

// ---- activation arithmetic, shared by the bandwidth kernels and the GEMM epilogues ----------
// Formulas follow the reference operation by operation (association order included):
//   LeakyReLU src/RMAD/LeakyReLUOperation.cs:54-93, Sigmoid src/RMAD/SigmoidOperation.cs:46-84,
//   Tanh src/RMAD/TanhOperation.cs:42-79, GELU src/RMAD/GELUOperation.cs:86-101,
//   AmplifiedSigmoid src/RMAD/AmplifiedSigmoidOperation.cs:44-84.
template <typename T> struct GeluConst;
template <> struct GeluConst<double> {
    // sqrt(2 / pi) in double
    static __device__ __forceinline__ double s() { return 0.79788456080286535588; }
    static __device__ __forceinline__ double c0() { return 0.044715; }
};
template <> struct GeluConst<float> {
    // PRADLite: (float)sqrt((double)(2 / (float)pi))
    static __device__ __forceinline__ float s() { return 0.797884523868560791015625f; }
    static __device__ __forceinline__ float c0() { return 0.044715f; }
};

__device__ __forceinline__ double dev_tanh(double x) { return tanh(x); }
// PRADLite evaluates Math.Tanh in double and rounds once to float.
__device__ __forceinline__ float dev_tanh(float x) { return (float)tanh((double)x); }
__device__ __forceinline__ double dev_exp(double x) { return exp(x); }
__device__ __forceinline__ float dev_exp(float x) { return (float)exp((double)x); }
// tanh for the GELU kernels, which would otherwise be bound by the math library's tanh instead of
// by memory: tanh|u| = (1 - t) / (1 + t) with t = exp(-2|u|); below 0.01 the difference 1 - t cancels,
// so a Taylor polynomial (next term ~1e-22 relative) takes over.  Relative error ~1e-15 in double.
__device__ __forceinline__ double gelu_tanh(double u) {
    const double a = fabs(u);
    double r;
    if (a < 0.01) {
        const double a2 = a * a;
        r = a * (1.0 + a2 * (-1.0 / 3.0 + a2 * (2.0 / 15.0 + a2 * (-17.0 / 315.0 + a2 * (62.0 / 2835.0)))));
    } else {
        const double t = exp(-2.0 * a);
        r = (1.0 - t) / (1.0 + t);
    }
    return copysign(r, u);
}
// PRADLite rounds a double tanh to float; evaluating in float is within 3e-7 of it, far inside the
// 1e-5 parity bar, and keeps the kernel memory-bound.
__device__ __forceinline__ float gelu_tanh(float u) {
    const float a = fabsf(u);
    float r;
    if (a < 0.01f) {
        const float a2 = a * a;
        r = a * (1.0f + a2 * (-1.0f / 3.0f + a2 * (2.0f / 15.0f)));
    } else {
        const float t = __expf(-2.0f * a);
        r = (1.0f - t) * __builtin_amdgcn_rcpf(1.0f + t);  // 1 + t is in (1, 2]: the reciprocal is good to an ulp
    }
    return copysignf(r, u);
}
// x^3 (the reference's pow(x, 3) is correctly rounded; the product is within one ulp of it).
__device__ __forceinline__ float gelu_cube(float x) { return x * x * x; }
__device__ __forceinline__ double gelu_cube(double x) { return x * x * x; }

// GELU as the reference writes it, 0.5 x (1 + tanh(u)) with u = sqrt(2/pi) (x + 0.044715 x^3) (src/RMAD/GELUOperation.cs:86-92),
// and the factor its Backward multiplies by (:94-101; as written there, not the derivative).
__device__ __forceinline__ double gelu_value(double x) {
    const double a = 0.5 * (1.0 + gelu_tanh(GeluConst<double>::s() * (x + (GeluConst<double>::c0() * gelu_cube(x)))));
    return a * x;
}
__device__ __forceinline__ double gelu_factor(double s) {
    const double b = gelu_tanh(GeluConst<double>::s() * (s + (GeluConst<double>::c0() * gelu_cube(s))));
    const double omb = 1.0 - b * b;
    const double c = omb * omb;
    const double d = GeluConst<double>::s() * ((GeluConst<double>::c0() * 3.0 * (s * s)) + 1.0);
    return (0.5 * s * ((c * d) + b)) + (0.5 * (1.0 + b));
}
// In float the same functions in as few instructions as they take (PRADLite evaluates them in double and rounds; both forms
// are within 5e-7 of that, far inside the 1e-5 parity bar).  Measured on this chip: vector instructions issued beside
// float or double MFMAs add their full time to the MFMAs' (wavefronts that only multiply and wavefronts that only issue
// v_fma_f32, on the same SIMDs, take the sum of their separate times; with bf16 MFMAs they take the maximum) - the float
// and double matrix instructions do not overlap with the vector unit, so every vector instruction of an epilogue is time
// the products do not get.  0.5 (1 + tanh u) = 1 / (1 + e^(-2u)), e^(-2u) = 2^(x (k1 + k2 x^2)) on the hardware
// exponential and reciprocal: seven instructions for the value, about twenty for the factor.
__device__ __forceinline__ float gelu_exp_minus_2u(float x, float x2, float limit) {
    const float k1 = -2.302208185195923f;   // -2 s log2(e), s = PRADLite's float sqrt(2/pi)
    const float k2 = -0.10294323414564133f;  // k1 * 0.044715f
    return __builtin_amdgcn_exp2f(fminf(x * __builtin_fmaf(k2, x2, k1), limit));
}
__device__ __forceinline__ float gelu_value(float x) {
    const float e = gelu_exp_minus_2u(x, x * x, INFINITY);
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}
__device__ __forceinline__ float gelu_factor(float s) {
    const float x2 = s * s;
    const float e = gelu_exp_minus_2u(s, x2, 126.0f);  // (bounded, so that (1 - e) / (1 + e) stays -1 instead of inf / inf)
    const float b = (1.0f - e) * __builtin_amdgcn_rcpf(1.0f + e);  // tanh u
    const float omb = 1.0f - b * b;
    const float c = omb * omb;
    const float d = __builtin_fmaf(0.10703221708536148f, x2, 0.7978845238685608f);  // s (3 * 0.044715f x^2 + 1)
    return __builtin_fmaf(0.5f * s, __builtin_fmaf(c, d, b), 0.5f * (1.0f + b));
}

// AmplifiedSigmoid: pow(b, -x) with b = (float)pi - 2 (PradMath.PI is a float, src/PRAD/PradMath.cs:20, and the
// subtraction a float one), evaluated as exp(-x * ln b).
template <typename T>
__device__ __forceinline__ T amp_pow_neg(T x) {
    const double ln_b = 0.13242442855180583;  // log(1.1415927410125732421875)
    return (T)exp(-(double)x * ln_b);
}

template <typename T>
__device__ __forceinline__ T act_forward(int act, T x, T alpha) {
    switch (act) {
        case ACT_LEAKYRELU: return x > (T)0 ? x : alpha * x;
        case ACT_SIGMOID: return (T)1 / ((T)1 + dev_exp(-x));
        case ACT_TANH: return dev_tanh(x);
        case ACT_GELU: return gelu_value(x);
        case ACT_AMPLIFIED_SIGMOID: return (T)1 / ((T)1 + amp_pow_neg<T>(x));
        default: return x;
    }
}

// Derivative factor act'(src): src is the cached input x (LeakyReLU, GELU, AmplifiedSigmoid) or output y (Sigmoid, Tanh).
template <typename T>
__device__ __forceinline__ T act_derivative(int act, T s, T alpha) {
    switch (act) {
        case ACT_LEAKYRELU: return s > (T)0 ? (T)1 : alpha;
        case ACT_SIGMOID: return s * ((T)1 - s);
        case ACT_TANH: return (T)1 - s * s;
        case ACT_GELU: return gelu_factor(s);
        case ACT_AMPLIFIED_SIGMOID: {  // as written: pow(b, -x) / pow(1 + pow(b, -x), 2), no ln(b) factor
            const T e = amp_pow_neg<T>(s);
            const T q = (T)1 + e;
            return e / (q * q);
        }
        default: return (T)1;
    }
}

// ---- GEMM launch description -------------------------------------------------------------
// C[M x N] (+)= op(A)[M x K] . op(B)[K x N], all row-major with leading dimensions in elements.
//   transA == 0: A is M x K (lda >= K);  transA == 1: A is K x M (lda >= M)
//   transB == 0: B is K x N (ldb >= N);  transB == 1: B is N x K (ldb >= K)
// Epilogue (applied to the finished accumulator v at (i, j), in this order):
//   v += bias[j]                      when bias != nullptr
//   if (Z) Z[i][j] = v                pre-activation copy
//   v = act_forward(act_fwd, v)       when act_fwd != ACT_NONE
//   v *= act_derivative(act_bwd, act_src[i][j])   when act_bwd != ACT_NONE
//   C[i][j] = accumulate ? C[i][j] + v : v
// batch > 1 runs `batch` independent products; strides are in elements (0 broadcasts).
template <typename T>
struct GemmArgs {
    int transA, transB;
    int64_t M, N, K;
    const T* A; int64_t lda;
    const T* B; int64_t ldb;
    T* C; int64_t ldc;
    int accumulate;
    const T* bias;
    T* Z; int64_t ldz;
    int act_fwd;
    int act_bwd;
    const T* act_src; int64_t ld_act;
    T alpha;
    int batch;
    int64_t strideA, strideB, strideC;
    // Two-level batches (windows x heads): with batch_inner > 1, product b takes operand blocks at
    // (b / batch_inner) * stride + (b % batch_inner) * istride.
    int batch_inner;
    int64_t istrideA, istrideB, istrideC;
    // When set, C is not written: each workgroup stores the sum of its finished tile to
    // tile_sums[batch_index * tiles_per_product + tile_index] (MatrixMultiplyAndSum forward).
    double* tile_sums;
    // Scratch for products that are split along K (see gemm_split_factor): split_ws holds
    // split_factor * batch * M * N elements.  Filled in by the caller; nullptr disables splitting.
    T* split_ws;
    // Set by launch_gemm for the kernels: K range per split (0 = not split) and the element offsets
    // of split z's operand blocks from those of split 0.
    int64_t ksplit;
    int64_t zstrideA, zstrideB;
    // One zeroed unsigned per tile and batch (left zeroed): with it, a product split along K (several ways, see
    // gemm_split_factor, or two ways, see gemm_pairs) runs as one launch in which the workgroup that arrives
    // last at a tile's counter adds the partial tiles; without it, a several-way split takes a second launch
    // and a product that would run as pairs runs unsplit.
    unsigned* split_counters;
    // Set by launch_gemm: the first shared_tiles tiles of the launch are each shared by shared_splits workgroups, a K
    // range each, while the tiles after them run unsplit in the same launch (see gemm_shared_tiles_plan).  Their
    // partial tiles lie compactly in split_ws, tile by tile.  0 = none.
    int shared_tiles, shared_splits;
    // LSTM step epilogues (launch_lstm_step_fwd / _bwd; see there).  All matrices are rows x lstm_hidden with
    // leading dimension lstm_hidden, except gates / dG (rows x 4 * lstm_hidden, blocks [i | f | g | o]).
    int64_t lstm_hidden;
    const T* lstm_c_prev; const T* lstm_tanh_c_in; const T* lstm_gates; const T* lstm_dh_loss; const T* lstm_dc_in;
    T* lstm_c; T* lstm_tanh_c; T* lstm_h; T* lstm_dG; T* lstm_dc_prev;
    // A sum of products C = sum_q op(A_q).op(B_q): nseg > 1 operand pairs, segstrideA / segstrideB
    // elements apart, M x K and K x N each.  Runs as a product split along the joint reduction
    // (one pair per split), so split_ws must hold nseg * M * N elements.  batch must be 1.
    int nseg;
    int64_t segstrideA, segstrideB;
    // A column sum that rides along with the product's launch (the bias gradient of
    // MatrixAddBroadcasting next to the weight gradient, both functions of the same upstream
    // gradient): colsum_dst[j] = sum_i colsum_src[i][j] over colsum_rows x colsum_cols, taken by extra
    // workgroups appended to the grid.  nullptr = none.  Only for colsum_rows below COLSUM_CHUNK_ROWS.
    const T* colsum_src;
    T* colsum_dst;
    int64_t colsum_rows, colsum_cols;
};

// Column sums of 64 columns [64 * bx, ...) over rows [r0, r1) by one workgroup of 256 threads (four
// wavefronts take every fourth row, four accumulators each); part is 4 x 64 doubles of LDS.
template <typename T, typename OUT>
__device__ __forceinline__ void colsum_block(const T* __restrict__ dy, OUT* __restrict__ out, int64_t cols, int64_t r0, int64_t r1,
                                             int64_t bx, double* part, int64_t pitch = 0) {
    if (pitch == 0) pitch = cols;  // (rows of dy are `pitch` elements apart)
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int64_t j = bx * 64 + lane;
    double acc0 = 0.0, acc1 = 0.0, acc2 = 0.0, acc3 = 0.0;
    if (j < cols) {
        int64_t i = r0 + w;
        // sixteen loads in flight where the rows allow; the additions keep the order of the four-at-a-time loop below
        for (; i + 60 < r1; i += 64) {
            double v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) v[u] = (double)dy[(i + 4 * u) * pitch + j];
#pragma unroll
            for (int u = 0; u < 16; u += 4) { acc0 += v[u]; acc1 += v[u + 1]; acc2 += v[u + 2]; acc3 += v[u + 3]; }
        }
        for (; i + 12 < r1; i += 16) {
            const double a = (double)dy[i * pitch + j], b = (double)dy[(i + 4) * pitch + j];
            const double c = (double)dy[(i + 8) * pitch + j], d = (double)dy[(i + 12) * pitch + j];
            acc0 += a; acc1 += b; acc2 += c; acc3 += d;
        }
        for (; i < r1; i += 4) acc0 += (double)dy[i * pitch + j];
    }
    part[w * 64 + lane] = (acc0 + acc1) + (acc2 + acc3);
    __syncthreads();
    if (w == 0 && j < cols) out[j] = (OUT)((part[lane] + part[64 + lane]) + (part[128 + lane] + part[192 + lane]));
}
constexpr int64_t COLSUM_CHUNK_ROWS = 2048;  // taller matrices are summed in row chunks by two launches

// How many ways launch_gemm splits the reduction of a product whose output has too few tiles to occupy
// the chip (1 = not split).  A split product writes its partial results to GemmArgs::split_ws and a
// second kernel adds them in split order and applies the epilogue.
int gemm_split_factor(int64_t M, int64_t N, int64_t K, int batch, int elem_size);
// Whether launch_gemm would run the product as pairs of workgroups per tile (needs GemmArgs::split_counters and
// split_ws: 2 * batch * M * N elements).  In-kernel reduction uses at most GEMM_SPLIT_MAX_TILES counters.
bool gemm_pairs(int64_t M, int64_t N, int64_t K, int batch, int elem_size);
// A^T . B with a very long K and a small output, float: one pass over both operands (csrc/gemm_skinny.hip).  The launch
// needs gemm_skinny_workspace_bytes() of split_ws (0: not such a product) and returns hipErrorNotSupported otherwise.
bool gemm_skinny_eligible(const GemmArgs<float>& a);
size_t gemm_skinny_workspace_bytes(const GemmArgs<float>& a);
hipError_t launch_gemm_skinny(const GemmArgs<float>& a, hipStream_t stream);
// A . op(B) in float with tens of thousands of rows and a right operand small enough to stay in LDS (csrc/gemm_tall.hip),
// any elementwise epilogue; returns hipErrorNotSupported for other products.
bool gemm_tall_eligible(const GemmArgs<float>& a);
hipError_t launch_gemm_tall(const GemmArgs<float>& a, hipStream_t stream);
// A product on 128 x 128 tiles whose tile count leaves a poorly filled last round of workgroups (576 tiles over 512
// workgroup slots: 64 tiles would run alone on 64 compute units while 192 sit idle) splits that many tiles along K
// so that they fill the chip too.  Returns how many ways (0: none) and, through shared_tiles, how many tiles;
// split_ws must then hold shared_tiles * ways * 128 * 128 elements and split_counters be set.
int gemm_shared_tiles_plan(int64_t M, int64_t N, int64_t K, int batch, int elem_size, int* shared_tiles);
constexpr int GEMM_SPLIT_MAX_TILES = 384;

// Number of 128 x 128 output tiles of one product (the tile_sums layout).
inline int64_t gemm_tiles_per_product(int64_t M, int64_t N) { return ((M + 127) / 128) * ((N + 127) / 128); }

template <typename T> hipError_t launch_gemm(const GemmArgs<T>& args, hipStream_t stream);
// first = dC . B^T (transB) and second = A^T . dC (transA, may carry the column-sum rider) in one launch;
// hipErrorNotSupported (nothing launched) unless each alone would run unsplit on tiles of the same size.
template <typename T> hipError_t launch_gemm_pair(const GemmArgs<T>& first, const GemmArgs<T>& second, hipStream_t stream);

// One LSTM time step forward in one launch: gates = act(C + A . B) with C (rows x 4H) holding the input
// projection plus bias, A = h_{t-1} (rows x H), B = W_h (H x 4H); then c = f.c_prev + i.g, tanh_c, h = o.tanh_c.
// The activated gates replace C.  A workgroup's tile gathers the four gate columns of 8 hidden units, so the
// cell arithmetic has all it needs.  Same arithmetic as the product followed by launch_lstm_cell_fwd.
// Returns hipErrorNotSupported for shapes it does not take (H not a multiple of the slab depth, unaligned
// operands): the caller then runs the two launches.
template <typename T> hipError_t launch_lstm_step_fwd(const GemmArgs<T>& args, hipStream_t stream);
// One LSTM time step backward in one launch: dh = dh_loss + A . B^T with A = dG_{t+1} (rows x 4H), B = W_h,
// then the cell's backward (as launch_lstm_cell_bwd) writes dG_t and dc_prev.  split_ws / split_counters as for
// launch_gemm.
template <typename T> hipError_t launch_lstm_step_bwd(const GemmArgs<T>& args, hipStream_t stream);

// ---- bandwidth kernels ----------------------------------------------------------------------
template <typename T> hipError_t launch_add(const T* a, const T* b, T* y, int64_t n, hipStream_t s);
template <typename T> hipError_t launch_add_three(const T* a, const T* b, const T* c, T* y, int64_t n, hipStream_t s);
template <typename T> hipError_t launch_transpose(const T* x, T* y, int64_t rows, int64_t cols, hipStream_t s);
template <typename T> hipError_t launch_layernorm_fwd(const T* x, T* y, T* mean, T* stddev, int64_t rows, int64_t cols, hipStream_t s);
template <typename T> hipError_t launch_layernorm_bwd(const T* x, const T* mean, const T* stddev, const T* dy, T* dx, int64_t rows,
                                                      int64_t cols, hipStream_t s);
template <typename T> hipError_t launch_act_fwd(int act, const T* x, T* y, int64_t n, T alpha, hipStream_t s);
template <typename T> hipError_t launch_act_bwd(int act, const T* src, const T* dy, T* dx, int64_t n, T alpha, hipStream_t s);
template <typename T> hipError_t launch_hadamard_fwd(const T* a, const T* b, T* y, int64_t n, hipStream_t s);
template <typename T> hipError_t launch_hadamard_bwd(const T* a, const T* b, const T* dy, T* da, T* db, int64_t n, hipStream_t s);
template <typename T> hipError_t launch_accumulate(T* dest, const T* grad, int64_t n, hipStream_t s);
template <typename T> hipError_t launch_copy(T* dst, const T* src, int64_t n, hipStream_t s);
template <typename T> hipError_t launch_scale(T* y, const T* x, int64_t n, T alpha, hipStream_t s);
template <typename T> hipError_t launch_add_broadcast_fwd(const T* x, const T* bias, T* y, int64_t rows, int64_t cols, hipStream_t s);
int colsum_chunks(int64_t rows);
template <typename T> hipError_t launch_colsum(const T* dy, T* db, int64_t rows, int64_t cols, double* workspace, hipStream_t s);
template <typename T> hipError_t launch_fill_zero(T* p, int64_t n, hipStream_t s);
// n regions (16-byte aligned, sizes multiples of 4 bytes) zeroed by one launch per ZERO_TABLE_MAX of them.
constexpr int ZERO_TABLE_MAX = 40;
hipError_t launch_fill_zero_multi(void* const* ptrs, const size_t* bytes, int n, hipStream_t s);

// Descriptor of one tensor of a multi-tensor clip / Adam launch.
template <typename T>
struct TensorDesc {
    T* g; T* w; T* m; T* v;
    int64_t n;
};
// Clip needs device workspace of clip_workspace_bytes(sizes, ntensors) bytes.  `host_descs` is read
// during the call only.  c1 = 1 / (1 - beta1^t), c2 = 1 / (1 - beta2^t), evaluated by the caller
// in T like the reference does.
size_t clip_workspace_bytes(const int64_t* n, int ntensors);
template <typename T> hipError_t launch_clip(const TensorDesc<T>* host_descs, int ntensors, void* workspace, T clip_value,
                                             T min_value, hipStream_t s);
// Called after every launch of the Adam kernel with the stream it went to (a recording notes the graph node there).
struct AdamLaunchObserver {
    void (*fn)(void* ctx, hipStream_t s);
    void* ctx;
};
// reverse: AdamOptimizer.ReverseAdamUpdate instead of UpdateWeightWithAdam
template <typename T> hipError_t launch_adam(const TensorDesc<T>* host_descs, int ntensors, T lr, T beta1, T beta2, T eps, T c1,
                                             T c2, bool reverse, hipStream_t s, const AdamLaunchObserver* obs = nullptr);
template <typename T> hipError_t launch_clip_adam(const TensorDesc<T>* host_descs, int ntensors, void* workspace, T clip_value,
                                                  T min_value, T lr, T beta1, T beta2, T eps, T c1, T c2, hipStream_t s,
                                                  const AdamLaunchObserver* obs = nullptr);
// Replaces c1 and c2 in the launch arguments of a recorded Adam kernel node of an instantiated graph.
template <typename T> hipError_t adam_node_set_bias_correction(hipGraphExec_t exec, hipGraphNode_t node, T c1, T c2);

// Reductions across a wavefront (a butterfly over lane distances 32, 16, ... 1) and the exponential of the short-row
// softmax kernels, shared by csrc/loss.hip and csrc/head.hip so that both give the same bits.
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ double wave_max(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmax(v, __shfl_xor(v, off, 64));
    return v;
}

// Reductions and exponentials in the element type for the short-row kernels: in float they move one register per
// shuffle step instead of two and use the hardware exponential (within 2e-7 of the double evaluation rounded to
// float, far inside the 1e-5 parity bar), which is what those kernels' time goes into.
__device__ __forceinline__ float wave_sum_t(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ double wave_sum_t(double v) { return wave_sum(v); }
__device__ __forceinline__ float wave_max_t(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ double wave_max_t(double v) { return wave_max(v); }
__device__ __forceinline__ float short_exp(float x) { return __expf(x); }
__device__ __forceinline__ double short_exp(double x) { return exp(x); }

// softmax / categorical cross-entropy (csrc/loss.hip)
template <typename T> hipError_t launch_softmax_fwd(const T* x, T* y, int64_t rows, int64_t cols, T alpha, hipStream_t s);
template <typename T> hipError_t launch_softmax_bwd(const T* y, const T* dy, T* dx, int64_t rows, int64_t cols, T alpha, hipStream_t s);
template <typename T> hipError_t launch_softmax_cce(const T* x, const T* t, T* y, T* dy, T* dx, T* loss, unsigned* counter, int64_t rows, int64_t cols, hipStream_t s);
template <typename T> hipError_t launch_cce_fwd(const T* p, const T* t, T* loss, int64_t rows, int64_t cols, hipStream_t s);
template <typename T> hipError_t launch_cce_bwd(const T* p, const T* t, T* dp, int64_t rows, int64_t cols, hipStream_t s);

// The output layer of a classifier with softmax and categorical cross-entropy, forward and backward, in one launch of one
// workgroup (csrc/head.hip): Z = A . W + bias, P = softmax(Z), loss, dP, dZ, then dbias, dW (+)= A^T . dZ and
// dA = dZ . W^T (.) act'(act_src).  All matrices dense row-major; Z, loss, dbias, dW, dA may be nullptr.
template <typename T>
struct HeadArgs {
    const T* A; const T* W; const T* bias; const T* target; const T* act_src;
    T* Z; T* P; T* loss; T* dP; T* dZ; T* dA; T* dW; T* dbias;
    int B, H, C;  // rows of the batch, inputs of the layer, classes
    int act;      // activation of the layer below (its Backward multiplies dA), ACT_NONE: none
    T alpha;
    int accumulate_dW;
};
template <typename T> bool classifier_head_eligible(int64_t B, int64_t H, int64_t C);
template <typename T> size_t classifier_head_lds_bytes(int64_t B, int64_t H, int64_t C);
// hipErrorNotSupported for shapes the kernel does not take (the caller then uses the separate launches).
template <typename T> hipError_t launch_classifier_head(const HeadArgs<T>& a, hipStream_t s);

size_t mse_workspace_bytes();
// dy != nullptr: the gradient is written in the same pass (the values of launch_mse_bwd).
template <typename T> hipError_t launch_mse_fwd(const T* y, const T* t, T* loss, double* workspace, int64_t n, hipStream_t s,
                                                T* dy = nullptr);
template <typename T> hipError_t launch_mse_bwd(const T* y, const T* t, T* dy, int64_t n, hipStream_t s);

// LSTM cell (csrc/lstm.hip)
template <typename T> hipError_t launch_lstm_cell_fwd(T* G, const T* c_prev, T* c, T* tanh_c, T* h, int64_t rows, int64_t hidden,
                                                      hipStream_t s);
template <typename T> hipError_t launch_lstm_cell_bwd(const T* gates, const T* c_prev, const T* tanh_c, const T* dh_a, const T* dh_b,
                                                      const T* dc_in, T* dG, T* dc_prev, int64_t rows, int64_t hidden, hipStream_t s);

// A whole LSTM sequence in one launch each way (csrc/lstm_seq.hip; float).
struct LstmSeqArgs {
    const float* Wh;   // hidden x 4*hidden, gate blocks [i | f | g | o]
    float* G;          // steps*batch x 4*hidden: pre-activations in, activated gates out (forward); gates in (backward)
    float* C;          // (steps+1)*batch x hidden, block 0 = c_0
    float* Hs;         // (steps+1)*batch x hidden, block 0 = h_0
    float* TC;         // steps*batch x hidden: tanh(c_t)
    const float* dHl;  // steps*batch x hidden: loss gradient with respect to h_t (backward)
    float* dG;         // steps*batch x 4*hidden (backward)
    float* partial;    // backward: lstm_seq_partial_bytes() of scratch
    unsigned* flags;   // (batch/16) * (hidden/16) words
    unsigned* abort_word;  // host-visible; a workgroup that gives up waiting writes 1
    int batch, hidden, steps;
    int spin_limit;
    int local;             // the probe found every row group on one XCD: the kernels may exchange through that XCD's L2
};
bool lstm_seq_eligible(int64_t batch, int64_t hidden, int64_t steps, int compute_units);
size_t lstm_seq_partial_bytes(int64_t batch, int64_t hidden);
hipError_t launch_lstm_seq(const LstmSeqArgs& a, bool backward, hipStream_t s);
bool lstm_seq_local(int64_t batch);
hipError_t launch_lstm_seq_probe(int64_t batch, int64_t hidden, unsigned* flags, unsigned* abort_word, int spin_limit, hipStream_t s);

// Windowed self-attention, forward, one launch (csrc/attention.hip; float, head dimension 32, <= 64 tokens per window)
bool window_attention_supported(int64_t tokens, int64_t head_dim);
hipError_t launch_window_attention_fwd(const float* QKV, float* P, float* O, int64_t windows, int64_t heads, int64_t tokens, float scale,
                                       hipStream_t stream);
hipError_t launch_window_attention_bwd(const float* QKV, const float* P, const float* dO, float* dQKV, int64_t windows, int64_t heads,
                                       int64_t tokens, float scale, hipStream_t stream);

// MatrixMultiplyAndSum
// S = samples of a batch (each with its own A, out, dOut, dA and P slices of dB; the P slices of B are shared).
template <typename T> hipError_t launch_matmul_sum_fwd(const T* A, const T* B, T* out, double* workspace, int64_t M, int64_t K,
                                                       int64_t N, int64_t P, int64_t S, hipStream_t s);
template <typename T> hipError_t launch_matmul_sum_bwd(const T* A, const T* B, const T* dOut, T* dA, T* dB, int64_t M, int64_t K,
                                                       int64_t N, int64_t P, int64_t S, hipStream_t s);

}  // namespace prad
