// Bandwidth-bound kernels around the matrix products: activation forward/backward
// (LeakyReLU, Sigmoid, Tanh, GELU), Hadamard product, gradient accumulation, bias broadcast and
// its column sum.  Each replaces a scalar double loop of the reference
// (src/RMAD/LeakyReLUOperation.cs:54-93, SigmoidOperation.cs:46-84, TanhOperation.cs:42-79,
// GELUOperation.cs:44-101, HadamardProductOperation.cs:50-118, OperationBase.cs:295-303,
// MatrixAddBroadcastingOperation.cs:32-70).
//
// Every kernel streams: a thread moves 16-byte vectors, a workgroup of 256 threads covers
// UNROLL consecutive 4 KiB blocks per step so that several independent loads are in flight per
// lane, and the grid is sized to the data (no tail workgroups spinning on a stride loop).
// a*b+c is never contracted here, to keep the reference's rounding of each operation.
#include "common.h"

#pragma clang fp contract(off)

namespace prad {

constexpr int EW_THREADS = 256;
constexpr int EW_UNROLL = 4;

template <typename T> struct Vec16;
template <> struct Vec16<double> { typedef double type __attribute__((ext_vector_type(2))); static constexpr int N = 2; };
template <> struct Vec16<float> { typedef float type __attribute__((ext_vector_type(4))); static constexpr int N = 4; };

// Generic streaming map: out_k[i] = f(in_0[i], ..., in_{NIN-1}[i]) for NOUT outputs.
// F::apply(const T (&in)[NIN], T (&out)[NOUT]).
template <typename T, int NIN, int NOUT>
struct StreamPtrs {
    const T* in[NIN];
    T* out[NOUT];
};

template <typename T, int NIN, int NOUT, typename F>
__global__ void __launch_bounds__(EW_THREADS) stream_kernel(StreamPtrs<T, NIN, NOUT> p, int64_t n, F f) {
    typedef typename Vec16<T>::type V;
    constexpr int VN = Vec16<T>::N;
    const int64_t nvec = n / VN;
    const int64_t base = ((int64_t)blockIdx.x * EW_UNROLL) * EW_THREADS + threadIdx.x;
    V vin[EW_UNROLL][NIN];
#pragma unroll
    for (int u = 0; u < EW_UNROLL; ++u) {
        const int64_t iv = base + (int64_t)u * EW_THREADS;
        if (iv < nvec) {
#pragma unroll
            for (int a = 0; a < NIN; ++a) vin[u][a] = __builtin_nontemporal_load(reinterpret_cast<const V*>(p.in[a]) + iv);
        }
    }
#pragma unroll
    for (int u = 0; u < EW_UNROLL; ++u) {
        const int64_t iv = base + (int64_t)u * EW_THREADS;
        if (iv < nvec) {
            V vout[NOUT];
#pragma unroll
            for (int e = 0; e < VN; ++e) {
                T in[NIN], out[NOUT];
#pragma unroll
                for (int a = 0; a < NIN; ++a) in[a] = vin[u][a][e];
                f.apply(in, out);
#pragma unroll
                for (int o = 0; o < NOUT; ++o) vout[o][e] = out[o];
            }
#pragma unroll
            for (int o = 0; o < NOUT; ++o) __builtin_nontemporal_store(vout[o], reinterpret_cast<V*>(p.out[o]) + iv);
        }
    }
    // Scalar tail (n not a multiple of the vector width): handled by the last workgroup.
    if (blockIdx.x == gridDim.x - 1) {
        const int64_t i = nvec * VN + threadIdx.x;
        if (i < n) {
            T in[NIN], out[NOUT];
#pragma unroll
            for (int a = 0; a < NIN; ++a) in[a] = p.in[a][i];
            f.apply(in, out);
#pragma unroll
            for (int o = 0; o < NOUT; ++o) p.out[o][i] = out[o];
        }
    }
}

// Scalar variant for buffers that are not 16-byte aligned (borrowed device memory).
template <typename T, int NIN, int NOUT, typename F>
__global__ void __launch_bounds__(EW_THREADS) stream_kernel_scalar(StreamPtrs<T, NIN, NOUT> p, int64_t n, F f) {
    for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < n; i += (int64_t)gridDim.x * EW_THREADS) {
        T in[NIN], out[NOUT];
#pragma unroll
        for (int a = 0; a < NIN; ++a) in[a] = p.in[a][i];
        f.apply(in, out);
#pragma unroll
        for (int o = 0; o < NOUT; ++o) p.out[o][i] = out[o];
    }
}

template <typename T, int NIN, int NOUT, typename F>
static hipError_t launch_stream(const StreamPtrs<T, NIN, NOUT>& p, int64_t n, F f, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    bool aligned = true;
    for (int a = 0; a < NIN; ++a) aligned = aligned && (reinterpret_cast<uintptr_t>(p.in[a]) % 16 == 0);
    for (int o = 0; o < NOUT; ++o) aligned = aligned && (reinterpret_cast<uintptr_t>(p.out[o]) % 16 == 0);
    if (aligned) {
        constexpr int VN = Vec16<T>::N;
        const int64_t nvec = n / VN;
        const int64_t per_block = (int64_t)EW_THREADS * EW_UNROLL;
        int64_t blocks = (nvec + per_block - 1) / per_block;
        if (blocks < 1) blocks = 1;
        hipLaunchKernelGGL((stream_kernel<T, NIN, NOUT, F>), dim3((unsigned)blocks), dim3(EW_THREADS), 0, s, p, n, f);
    } else {
        int64_t blocks = (n + EW_THREADS - 1) / EW_THREADS;
        if (blocks > 65536) blocks = 65536;
        hipLaunchKernelGGL((stream_kernel_scalar<T, NIN, NOUT, F>), dim3((unsigned)blocks), dim3(EW_THREADS), 0, s, p, n, f);
    }
    return hipGetLastError();
}

// ---- functors ---------------------------------------------------------------------------
template <typename T, int ACT> struct ActFwd {
    T alpha;
    __device__ __forceinline__ void apply(const T (&in)[1], T (&out)[1]) const { out[0] = act_forward<T>(ACT, in[0], alpha); }
};
template <typename T, int ACT> struct ActBwd {  // in: src, dy
    T alpha;
    __device__ __forceinline__ void apply(const T (&in)[2], T (&out)[1]) const {
        out[0] = in[1] * act_derivative<T>(ACT, in[0], alpha);
    }
};
template <typename T> struct HadFwd {
    __device__ __forceinline__ void apply(const T (&in)[2], T (&out)[1]) const { out[0] = in[0] * in[1]; }
};
template <typename T> struct HadBwd {  // in: a, b, dy ; out: da, db
    __device__ __forceinline__ void apply(const T (&in)[3], T (&out)[2]) const {
        out[0] = in[2] * in[1];
        out[1] = in[2] * in[0];
    }
};
template <typename T> struct Scale {
    T alpha;
    __device__ __forceinline__ void apply(const T (&in)[1], T (&out)[1]) const { out[0] = in[0] * alpha; }
};
template <typename T> struct Copy {
    __device__ __forceinline__ void apply(const T (&in)[1], T (&out)[1]) const { out[0] = in[0]; }
};
template <typename T> struct Add2 {  // MatrixAddOperation, src/RMAD/MatrixAddOperation.cs:30-45
    __device__ __forceinline__ void apply(const T (&in)[2], T (&out)[1]) const { out[0] = in[0] + in[1]; }
};
template <typename T> struct Add3 {  // MatrixAddThreeOperation, src/RMAD/MatrixAddThreeOperation.cs:35-50: (a + b) + c
    __device__ __forceinline__ void apply(const T (&in)[3], T (&out)[1]) const { out[0] = (in[0] + in[1]) + in[2]; }
};
template <typename T> struct Accum {  // in: dest, grad ; out: dest
    __device__ __forceinline__ void apply(const T (&in)[2], T (&out)[1]) const { out[0] = in[0] + in[1]; }
};

template <typename T>
hipError_t launch_act_fwd(int act, const T* x, T* y, int64_t n, T alpha, hipStream_t s) {
    StreamPtrs<T, 1, 1> p{{x}, {y}};
    switch (act) {
        case ACT_LEAKYRELU: return launch_stream(p, n, ActFwd<T, ACT_LEAKYRELU>{alpha}, s);
        case ACT_SIGMOID: return launch_stream(p, n, ActFwd<T, ACT_SIGMOID>{alpha}, s);
        case ACT_TANH: return launch_stream(p, n, ActFwd<T, ACT_TANH>{alpha}, s);
        case ACT_GELU: return launch_stream(p, n, ActFwd<T, ACT_GELU>{alpha}, s);
        case ACT_AMPLIFIED_SIGMOID: return launch_stream(p, n, ActFwd<T, ACT_AMPLIFIED_SIGMOID>{alpha}, s);
        default: return hipErrorInvalidValue;
    }
}
template <typename T>
hipError_t launch_act_bwd(int act, const T* src, const T* dy, T* dx, int64_t n, T alpha, hipStream_t s) {
    StreamPtrs<T, 2, 1> p{{src, dy}, {dx}};
    switch (act) {
        case ACT_LEAKYRELU: return launch_stream(p, n, ActBwd<T, ACT_LEAKYRELU>{alpha}, s);
        case ACT_SIGMOID: return launch_stream(p, n, ActBwd<T, ACT_SIGMOID>{alpha}, s);
        case ACT_TANH: return launch_stream(p, n, ActBwd<T, ACT_TANH>{alpha}, s);
        case ACT_GELU: return launch_stream(p, n, ActBwd<T, ACT_GELU>{alpha}, s);
        case ACT_AMPLIFIED_SIGMOID: return launch_stream(p, n, ActBwd<T, ACT_AMPLIFIED_SIGMOID>{alpha}, s);
        default: return hipErrorInvalidValue;
    }
}
template <typename T>
hipError_t launch_hadamard_fwd(const T* a, const T* b, T* y, int64_t n, hipStream_t s) {
    StreamPtrs<T, 2, 1> p{{a, b}, {y}};
    return launch_stream(p, n, HadFwd<T>{}, s);
}
template <typename T>
hipError_t launch_hadamard_bwd(const T* a, const T* b, const T* dy, T* da, T* db, int64_t n, hipStream_t s) {
    StreamPtrs<T, 3, 2> p{{a, b, dy}, {da, db}};
    return launch_stream(p, n, HadBwd<T>{}, s);
}
template <typename T>
hipError_t launch_add(const T* a, const T* b, T* y, int64_t n, hipStream_t s) {
    StreamPtrs<T, 2, 1> p{{a, b}, {y}};
    return launch_stream(p, n, Add2<T>{}, s);
}
template <typename T>
hipError_t launch_add_three(const T* a, const T* b, const T* c, T* y, int64_t n, hipStream_t s) {
    StreamPtrs<T, 3, 1> p{{a, b, c}, {y}};
    return launch_stream(p, n, Add3<T>{}, s);
}
template <typename T>
hipError_t launch_accumulate(T* dest, const T* grad, int64_t n, hipStream_t s) {
    StreamPtrs<T, 2, 1> p{{dest, grad}, {dest}};
    return launch_stream(p, n, Accum<T>{}, s);
}

// MatrixMultiplyScalarOperation (src/RMAD/MatrixMultiplyScalarOperation.cs): y = x * scalar, both directions.
template <typename T>
hipError_t launch_scale(T* y, const T* x, int64_t n, T alpha, hipStream_t s) {
    StreamPtrs<T, 1, 1> p{{x}, {y}};
    return launch_stream(p, n, Scale<T>{alpha}, s);
}

template <typename T>
hipError_t launch_copy(T* dst, const T* src, int64_t n, hipStream_t s) {
    StreamPtrs<T, 1, 1> p{{src}, {dst}};
    return launch_stream(p, n, Copy<T>{}, s);
}

// ---- zero fill (a kernel, so it can be recorded into a captured graph) --------------------
template <typename T>
__global__ void __launch_bounds__(EW_THREADS) fill_zero_kernel(T* p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < n; i += (int64_t)gridDim.x * EW_THREADS) p[i] = (T)0;
}
template <typename T>
hipError_t launch_fill_zero(T* p, int64_t n, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    int64_t blocks = (n + EW_THREADS - 1) / EW_THREADS;
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL((fill_zero_kernel<T>), dim3((unsigned)blocks), dim3(EW_THREADS), 0, s, p, n);
    return hipGetLastError();
}

// Several tensors zeroed by one launch (GradientClearer over a model's layers): a table of up to ZERO_TABLE_MAX regions as a
// kernel argument, cut into chunks of 16 KB; a workgroup finds its region by walking the table.
struct ZeroTable {
    unsigned char* ptr[ZERO_TABLE_MAX];
    unsigned long long bytes[ZERO_TABLE_MAX];
    unsigned first_chunk[ZERO_TABLE_MAX + 1];
    int n;
};
constexpr unsigned ZERO_CHUNK = 16384;
__global__ void __launch_bounds__(EW_THREADS) fill_zero_multi_kernel(const ZeroTable tab) {
    int t = 0;
    while (t + 1 < tab.n && blockIdx.x >= tab.first_chunk[t + 1]) ++t;
    const unsigned long long begin = (unsigned long long)(blockIdx.x - tab.first_chunk[t]) * ZERO_CHUNK;
    const unsigned long long end = min(begin + ZERO_CHUNK, tab.bytes[t]);
    unsigned char* base = tab.ptr[t];
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    const u4 z = {0u, 0u, 0u, 0u};
    unsigned long long at = begin + 16ull * threadIdx.x;  // (regions start 16-byte aligned, their sizes are multiples of 4 bytes)
    for (; at + 16 <= end; at += 16ull * EW_THREADS) *reinterpret_cast<u4*>(base + at) = z;
    if (at < end)
        for (unsigned long long b = at; b < end; b += 4) *reinterpret_cast<unsigned*>(base + b) = 0u;
}
hipError_t launch_fill_zero_multi(void* const* ptrs, const size_t* bytes, int n, hipStream_t s) {
    for (int g0 = 0; g0 < n; g0 += ZERO_TABLE_MAX) {
        ZeroTable tab{};
        tab.n = 0;
        unsigned chunks = 0;
        for (int i = g0; i < n && tab.n < ZERO_TABLE_MAX; ++i) {
            if (bytes[i] == 0) continue;
            if (reinterpret_cast<uintptr_t>(ptrs[i]) % 16 != 0 || bytes[i] % 4 != 0) return hipErrorInvalidValue;
            tab.ptr[tab.n] = static_cast<unsigned char*>(ptrs[i]);
            tab.bytes[tab.n] = bytes[i];
            tab.first_chunk[tab.n] = chunks;
            chunks += (unsigned)((bytes[i] + ZERO_CHUNK - 1) / ZERO_CHUNK);
            ++tab.n;
        }
        if (tab.n == 0) continue;
        tab.first_chunk[tab.n] = chunks;
        hipLaunchKernelGGL(fill_zero_multi_kernel, dim3(chunks), dim3(EW_THREADS), 0, s, tab);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    }
    return hipSuccess;
}

// ---- bias broadcast: y[i][j] = x[i][j] + bias[j] -----------------------------------------
template <typename T>
__global__ void __launch_bounds__(EW_THREADS) add_broadcast_kernel(const T* __restrict__ x, const T* __restrict__ bias,
                                                                   T* __restrict__ y, int64_t rows, int64_t cols) {
    const int64_t n = rows * cols;
    for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < n; i += (int64_t)gridDim.x * EW_THREADS)
        y[i] = x[i] + bias[i % cols];
}
template <typename T>
hipError_t launch_add_broadcast_fwd(const T* x, const T* bias, T* y, int64_t rows, int64_t cols, hipStream_t s) {
    const int64_t n = rows * cols;
    if (n <= 0) return hipSuccess;
    int64_t blocks = (n + EW_THREADS - 1) / EW_THREADS;
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL((add_broadcast_kernel<T>), dim3((unsigned)blocks), dim3(EW_THREADS), 0, s, x, bias, y, rows, cols);
    return hipGetLastError();
}

// ---- bias gradient: db[j] = sum_i dy[i][j], accumulated in double and rounded once (LINQ Sum over
// Column(j), which for float accumulates in double).  A workgroup owns 64 columns; its four
// wavefronts take rows i = w, w+4, w+8, ... with four independent loads in flight each, and the four
// partial sums are added in wavefront order, so the result does not depend on timing.  Neighbouring
// lanes read neighbouring columns: every row is one coalesced read.  Tall matrices (a whole sequence of
// gate gradients) are cut into row chunks whose partial sums a second pass adds (see colsum_chunks).
// Rows [blockIdx.y * rows_per_chunk, ...) of 64 columns; out is db itself (one chunk) or a row of partial sums.
template <typename T, typename OUT>
__global__ void __launch_bounds__(256) colsum_kernel(const T* __restrict__ dy, OUT* __restrict__ out, int64_t rows, int64_t cols,
                                                     int64_t rows_per_chunk) {
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_chunk;
    const int64_t r1 = min(rows, r0 + rows_per_chunk);
    __shared__ double part[4 * 64];
    colsum_block<T, OUT>(dy, out + (int64_t)blockIdx.y * cols, cols, r0, r1, blockIdx.x, part);
}
// Tall matrices are summed in row chunks of at least 64 rows (up to 256 chunks, so that the first stage fills the
// chip); the chunk sums, a chunks x cols matrix of doubles, are then summed by the same kernel.
int colsum_chunks(int64_t rows) {
    if (rows < COLSUM_CHUNK_ROWS) return 1;
    const int64_t c = rows / 64;
    return (int)(c > 256 ? 256 : c);
}
// workspace: colsum_chunks(rows) * cols doubles when colsum_chunks(rows) > 1.
template <typename T>
hipError_t launch_colsum(const T* dy, T* db, int64_t rows, int64_t cols, double* workspace, hipStream_t s) {
    if (cols <= 0) return hipSuccess;
    const int chunks = workspace != nullptr ? colsum_chunks(rows) : 1;
    const unsigned gx = (unsigned)((cols + 63) / 64);
    if (chunks == 1) {
        hipLaunchKernelGGL((colsum_kernel<T, T>), dim3(gx, 1), dim3(256), 0, s, dy, db, rows, cols, rows);
    } else {
        const int64_t per = (rows + chunks - 1) / chunks;
        hipLaunchKernelGGL((colsum_kernel<T, double>), dim3(gx, (unsigned)chunks), dim3(256), 0, s, dy, workspace, rows, cols, per);
        hipLaunchKernelGGL((colsum_kernel<double, T>), dim3(gx, 1), dim3(256), 0, s, workspace, db, (int64_t)chunks, cols,
                           (int64_t)chunks);
    }
    return hipGetLastError();
}

#define INSTANTIATE(T)                                                                                             \
    template hipError_t launch_act_fwd<T>(int, const T*, T*, int64_t, T, hipStream_t);                             \
    template hipError_t launch_act_bwd<T>(int, const T*, const T*, T*, int64_t, T, hipStream_t);                   \
    template hipError_t launch_hadamard_fwd<T>(const T*, const T*, T*, int64_t, hipStream_t);                      \
    template hipError_t launch_hadamard_bwd<T>(const T*, const T*, const T*, T*, T*, int64_t, hipStream_t);        \
    template hipError_t launch_add<T>(const T*, const T*, T*, int64_t, hipStream_t);                               \
    template hipError_t launch_add_three<T>(const T*, const T*, const T*, T*, int64_t, hipStream_t);               \
    template hipError_t launch_accumulate<T>(T*, const T*, int64_t, hipStream_t);                                  \
    template hipError_t launch_copy<T>(T*, const T*, int64_t, hipStream_t);                                        \
    template hipError_t launch_scale<T>(T*, const T*, int64_t, T, hipStream_t);                                    \
    template hipError_t launch_add_broadcast_fwd<T>(const T*, const T*, T*, int64_t, int64_t, hipStream_t);        \
    template hipError_t launch_colsum<T>(const T*, T*, int64_t, int64_t, double*, hipStream_t);                             \
    template hipError_t launch_fill_zero<T>(T*, int64_t, hipStream_t);
INSTANTIATE(double)
INSTANTIATE(float)

}  // namespace prad
