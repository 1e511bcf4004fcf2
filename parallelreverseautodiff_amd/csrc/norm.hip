// Operations that sit next to the matrix products in the reference's example graphs and keep a layer's
// activations on the device: MatrixTransposeOperation (src/RMAD/MatrixTransposeOperation.cs:30-64) and
// LayerNormalizationOperation (src/RMAD/LayerNormalizationOperation.cs:56-110).  Both are bound by
// memory: the transpose moves 2 element sizes per element through a 64 x 64 LDS tile so that reads
// and writes both walk rows; layer normalisation reads a row once into registers (rows up to 16 Ki
// elements) for mean, deviation and output, 2 element sizes per element forward, 3 backward.
#include "common.h"

#include <cstdlib>
#include <initializer_list>

#pragma clang fp contract(off)

namespace prad {

constexpr int TT = 64;  // transpose tile edge

template <typename T>
__global__ void __launch_bounds__(256) transpose_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t rows, int64_t cols) {
    __shared__ T tile[TT][TT + 1];
    // Tiles are walked along diagonals: with power-of-two row lengths, workgroups that run at the same time
    // would otherwise all write to rows a multiple of the same large stride apart, i.e. to the same memory channels.
    const int64_t by = (blockIdx.y + blockIdx.x) % gridDim.y;
    const int64_t r0 = by * TT, c0 = (int64_t)blockIdx.x * TT;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    T v[TT / 4];  // all 16 loads of a thread are issued before the first is used
#pragma unroll
    for (int e = 0; e < TT / 4; ++e) {
        const int64_t i = r0 + ty + 4 * e, j = c0 + tx;
        v[e] = (i < rows && j < cols) ? __builtin_nontemporal_load(x + i * cols + j) : (T)0;
    }
#pragma unroll
    for (int e = 0; e < TT / 4; ++e) tile[ty + 4 * e][tx] = v[e];
    __syncthreads();
#pragma unroll
    for (int e = 0; e < TT / 4; ++e) {
        const int r = ty + 4 * e;
        const int64_t i = c0 + r, j = r0 + tx;  // y is cols x rows
        if (i < cols && j < rows) __builtin_nontemporal_store(tile[tx][r], y + i * rows + j);
    }
}

template <typename T> struct NormVec;
template <> struct NormVec<double> { typedef double type __attribute__((ext_vector_type(2))); static constexpr int N = 2; };
template <> struct NormVec<float> { typedef float type __attribute__((ext_vector_type(4))); static constexpr int N = 4; };

// The same through 16-byte loads and stores, for matrices whose rows and columns are whole vectors: a tile of
// TR rows x TC columns of x becomes TC rows x TR columns of y.
template <typename T, int TR, int TC>
__global__ void __launch_bounds__(256) transpose_vec_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t rows, int64_t cols) {
    typedef typename NormVec<T>::type V;
    constexpr int VEC = NormVec<T>::N;
    constexpr int IN_VPR = TC / VEC, IN_ROWS = 256 / IN_VPR, IN_PASSES = TR / IN_ROWS;     // loads: vectors along x's columns
    constexpr int OUT_VPR = TR / VEC, OUT_ROWS = 256 / OUT_VPR, OUT_PASSES = TC / OUT_ROWS;  // stores: along x's rows
    __shared__ T tile[TR][TC + 1];
    // Diagonal order as above, with consecutive workgroups going down x's rows, i.e. along y's rows: what is
    // written at one time lies close together (measured: 74 % of the memory's peak against 70 % the other way).
    const int64_t r0 = (int64_t)blockIdx.x * TR, c0 = (int64_t)((blockIdx.y + blockIdx.x) % gridDim.y) * TC;
    const int t = threadIdx.x;
    V v[IN_PASSES];
#pragma unroll
    for (int e = 0; e < IN_PASSES; ++e) {
        const int64_t i = r0 + t / IN_VPR + e * IN_ROWS, j = c0 + (t % IN_VPR) * VEC;
        if (i < rows && j < cols) v[e] = __builtin_nontemporal_load(reinterpret_cast<const V*>(x + i * cols + j));
        else v[e] = (V)(T)0;
    }
#pragma unroll
    for (int e = 0; e < IN_PASSES; ++e)
#pragma unroll
        for (int k = 0; k < VEC; ++k) tile[t / IN_VPR + e * IN_ROWS][(t % IN_VPR) * VEC + k] = v[e][k];
    __syncthreads();
#pragma unroll
    for (int e = 0; e < OUT_PASSES; ++e) {
        const int c = t / OUT_VPR + e * OUT_ROWS, rv = (t % OUT_VPR) * VEC;
        const int64_t i = c0 + c, j = r0 + rv;  // y is cols x rows
        V o;
#pragma unroll
        for (int k = 0; k < VEC; ++k) o[k] = tile[rv + k][c];
        if (i < cols && j < rows) __builtin_nontemporal_store(o, reinterpret_cast<V*>(y + i * rows + j));
    }
}

template <typename T, int TR, int TC>
static hipError_t launch_transpose_vec(const T* x, T* y, int64_t rows, int64_t cols, hipStream_t s) {
    const int64_t gx = (rows + TR - 1) / TR, gy = (cols + TC - 1) / TC;
    if (gy > 65535 || gx > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL((transpose_vec_kernel<T, TR, TC>), dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, x, y, rows, cols);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_transpose(const T* x, T* y, int64_t rows, int64_t cols, hipStream_t s) {
    if (rows <= 0 || cols <= 0) return hipSuccess;
    constexpr int VEC = NormVec<T>::N;
    if (rows % VEC == 0 && cols % VEC == 0 && (cols + 63) / 64 <= 65535 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(y) % 16 == 0) {
        // 512-byte row segments on the side written (measured best of 32..128 x 64..256 tiles in either order)
        return launch_transpose_vec<T, 512 / (int)sizeof(T), 64>(x, y, rows, cols, s);
    }
    const int64_t gx = (cols + TT - 1) / TT, gy = (rows + TT - 1) / TT;
    if (gy > 65535) return hipErrorInvalidValue;
    hipLaunchKernelGGL((transpose_kernel<T>), dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, x, y, rows, cols);
    return hipGetLastError();
}

__device__ __forceinline__ double wave_sum_d(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// One wavefront per row, four rows per workgroup.  The reference sums a row left to right (LINQ Average and
// Sum, in double also for float rows); here every lane sums its strided share in double and the lanes are
// combined pairwise: same quantities, different association, inside the parity tolerance.  A row of up to
// 64 * LN_REGS elements is read once and kept in registers; longer rows are read three times.
constexpr int LN_REGS = 16;

template <typename T>
__global__ void __launch_bounds__(256) layernorm_fwd_kernel(const T* __restrict__ x, T* __restrict__ y, T* __restrict__ mean,
                                                            T* __restrict__ stddev, int64_t rows, int64_t cols) {
    const int64_t i = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= rows) return;
    const int lane = threadIdx.x & 63;
    const T* __restrict__ xr = x + i * cols;
    T* __restrict__ yr = y + i * cols;
    const T eps = (T)1e-9;
    if (cols <= 64 * LN_REGS) {
        T v[LN_REGS];
        double s = 0.0;
#pragma unroll
        for (int e = 0; e < LN_REGS; ++e) {
            const int64_t j = lane + 64 * e;
            v[e] = j < cols ? xr[j] : (T)0;
            s += (double)v[e];
        }
        const T m = (T)(wave_sum_d(s) / (double)cols);
        double q = 0.0;
#pragma unroll
        for (int e = 0; e < LN_REGS; ++e) {
            const int64_t j = lane + 64 * e;
            const T d = v[e] - m;
            if (j < cols) q += (double)(d * d);
        }
        const T sd = (T)sqrt((double)((T)wave_sum_d(q) / (T)cols));
        if (lane == 0) { mean[i] = m; stddev[i] = sd; }
#pragma unroll
        for (int e = 0; e < LN_REGS; ++e) {
            const int64_t j = lane + 64 * e;
            if (j < cols) yr[j] = (v[e] - m) / (sd + eps);
        }
        return;
    }
    double s = 0.0;
    for (int64_t j = lane; j < cols; j += 64) s += (double)xr[j];
    const T m = (T)(wave_sum_d(s) / (double)cols);
    double q = 0.0;
    for (int64_t j = lane; j < cols; j += 64) { const T d = xr[j] - m; q += (double)(d * d); }
    const T sd = (T)sqrt((double)((T)wave_sum_d(q) / (T)cols));
    if (lane == 0) { mean[i] = m; stddev[i] = sd; }
    for (int64_t j = lane; j < cols; j += 64) yr[j] = (xr[j] - m) / (sd + eps);
}

// Long rows: one workgroup per row, the row (up to 256 * LN_WG_REGS elements) held in registers.
constexpr int LN_WG_REGS = 32;

__device__ __forceinline__ double block_sum_d(double v, double* red) {
    v = wave_sum_d(v);
    __syncthreads();  // red may still be read from the previous use
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}


// VN = elements per access: NormVec<T>::N (16-byte vectors; needs cols % VN == 0 and 16-byte aligned pointers) or 1.
template <typename T, int VN>
__global__ void __launch_bounds__(256) layernorm_fwd_row_kernel(const T* __restrict__ x, T* __restrict__ y, T* __restrict__ mean,
                                                                T* __restrict__ stddev, int64_t rows, int64_t cols) {
    typedef T V __attribute__((ext_vector_type(VN)));
    constexpr int NVEC = LN_WG_REGS / VN;
    __shared__ double red[4];
    const int64_t i = blockIdx.x;
    const V* __restrict__ xr = reinterpret_cast<const V*>(x + i * cols);
    V* __restrict__ yr = reinterpret_cast<V*>(y + i * cols);
    const int64_t nv = cols / VN;
    const T eps = (T)1e-9;
    V v[NVEC];
    double s = 0.0;
#pragma unroll
    for (int e = 0; e < NVEC; ++e) {
        const int64_t j = threadIdx.x + 256 * e;
        if (j < nv) v[e] = __builtin_nontemporal_load(xr + j);
        else
#pragma unroll
            for (int c = 0; c < VN; ++c) v[e][c] = (T)0;
    }
#pragma unroll
    for (int e = 0; e < NVEC; ++e)
#pragma unroll
        for (int c = 0; c < VN; ++c) s += (double)v[e][c];
    const T m = (T)(block_sum_d(s, red) / (double)cols);
    double q = 0.0;
#pragma unroll
    for (int e = 0; e < NVEC; ++e) {
        const int64_t j = threadIdx.x + 256 * e;
        if (j < nv)
#pragma unroll
            for (int c = 0; c < VN; ++c) { const T d = v[e][c] - m; q += (double)(d * d); }
    }
    const T sd = (T)sqrt((double)((T)block_sum_d(q, red) / (T)cols));
    if (threadIdx.x == 0) { mean[i] = m; stddev[i] = sd; }
#pragma unroll
    for (int e = 0; e < NVEC; ++e) {
        const int64_t j = threadIdx.x + 256 * e;
        if (j < nv) {
            V o;
#pragma unroll
            for (int c = 0; c < VN; ++c) o[c] = (v[e][c] - m) / (sd + eps);
            __builtin_nontemporal_store(o, yr + j);
        }
    }
}

// As written in the reference (the diagonal of the Jacobian only):
// dx = dy * ((1 - 1/cols) / (sd + eps) - (x - mean)^2 / (cols * (sd + eps)^3)).
template <typename T>
__global__ void __launch_bounds__(256) layernorm_bwd_kernel(const T* __restrict__ x, const T* __restrict__ mean,
                                                            const T* __restrict__ stddev, const T* __restrict__ dy, T* __restrict__ dx,
                                                            int64_t rows, int64_t cols) {
    const int64_t i = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= rows) return;
    const int lane = threadIdx.x & 63;
    const T eps = (T)1e-9;
    const T m = mean[i], sde = stddev[i] + eps;
    const T inv = (T)1 / sde;
    const T exp1 = ((T)1 - ((T)1 / (T)cols)) * inv;
    const T denom = (T)cols * (sde * sde * sde);
    const T* __restrict__ xr = x + i * cols;
    const T* __restrict__ gr = dy + i * cols;
    T* __restrict__ dr = dx + i * cols;
    for (int64_t j = lane; j < cols; j += 64) {
        const T d = xr[j] - m;
        dr[j] = gr[j] * (exp1 - (d * d) / denom);
    }
}

// Backward over the flat matrix (rows * cols below 2^31): a thread takes four elements 256 apart, several times
// over, and looks its row's statistics up; every access is coalesced whatever the row length.
template <typename T, int VN>
__global__ void __launch_bounds__(256) layernorm_bwd_flat_kernel(const T* __restrict__ x, const T* __restrict__ mean,
                                                                 const T* __restrict__ stddev, const T* __restrict__ dy,
                                                                 T* __restrict__ dx, unsigned n, unsigned cols) {
    typedef T V __attribute__((ext_vector_type(VN)));
    constexpr int PER = 4;  // accesses per thread
    const T eps = (T)1e-9;
    const T colsT = (T)cols, frac = (T)1 - ((T)1 / (T)cols);
    const unsigned nv = n / VN;
    const unsigned base = blockIdx.x * (256u * PER) + threadIdx.x;
    const V* __restrict__ xv = reinterpret_cast<const V*>(x);
    const V* __restrict__ gv = reinterpret_cast<const V*>(dy);
    V* __restrict__ ov = reinterpret_cast<V*>(dx);
    V a[PER], g[PER];
#pragma unroll
    for (int e = 0; e < PER; ++e) {
        const unsigned iv = base + 256u * e;
        if (iv < nv) { a[e] = __builtin_nontemporal_load(xv + iv); g[e] = __builtin_nontemporal_load(gv + iv); }
    }
#pragma unroll
    for (int e = 0; e < PER; ++e) {
        const unsigned iv = base + 256u * e;
        if (iv < nv) {
            const unsigned i = (iv * VN) / cols;  // a vector never straddles rows: cols is a multiple of VN
            const T m = mean[i], sde = stddev[i] + eps;
            const T exp1 = frac * ((T)1 / sde);
            const T denom = colsT * (sde * sde * sde);
            V o;
#pragma unroll
            for (int c = 0; c < VN; ++c) { const T d = a[e][c] - m; o[c] = g[e][c] * (exp1 - (d * d) / denom); }
            __builtin_nontemporal_store(o, ov + iv);
        }
    }
}

template <typename T>
static bool norm_vector_ok(int64_t cols, std::initializer_list<const void*> ptrs) {
    if (cols % NormVec<T>::N != 0) return false;
    for (const void* p : ptrs) if (reinterpret_cast<uintptr_t>(p) % 16 != 0) return false;
    return true;
}

template <typename T>
hipError_t launch_layernorm_fwd(const T* x, T* y, T* mean, T* stddev, int64_t rows, int64_t cols, hipStream_t s) {
    if (rows <= 0 || cols <= 0) return hipSuccess;
    if (cols > 64 * LN_REGS && cols <= 256 * LN_WG_REGS && rows <= 0x7fffffffLL) {
        if (norm_vector_ok<T>(cols, {x, y}))
            hipLaunchKernelGGL((layernorm_fwd_row_kernel<T, NormVec<T>::N>), dim3((unsigned)rows), dim3(256), 0, s, x, y, mean, stddev,
                               rows, cols);
        else
            hipLaunchKernelGGL((layernorm_fwd_row_kernel<T, 1>), dim3((unsigned)rows), dim3(256), 0, s, x, y, mean, stddev, rows, cols);
        return hipGetLastError();
    }
    hipLaunchKernelGGL((layernorm_fwd_kernel<T>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, x, y, mean, stddev, rows, cols);
    return hipGetLastError();
}
template <typename T>
hipError_t launch_layernorm_bwd(const T* x, const T* mean, const T* stddev, const T* dy, T* dx, int64_t rows, int64_t cols,
                                hipStream_t s) {
    if (rows <= 0 || cols <= 0) return hipSuccess;
    if (rows * cols < 0x7fffffffLL) {
        const unsigned n = (unsigned)(rows * cols);
        if (norm_vector_ok<T>(cols, {x, dy, dx})) {
            const unsigned nv = n / NormVec<T>::N;
            hipLaunchKernelGGL((layernorm_bwd_flat_kernel<T, NormVec<T>::N>), dim3((nv + 1023u) / 1024u), dim3(256), 0, s, x, mean, stddev,
                               dy, dx, n, (unsigned)cols);
        } else {
            hipLaunchKernelGGL((layernorm_bwd_flat_kernel<T, 1>), dim3((n + 1023u) / 1024u), dim3(256), 0, s, x, mean, stddev, dy, dx, n,
                               (unsigned)cols);
        }
        return hipGetLastError();
    }
    hipLaunchKernelGGL((layernorm_bwd_kernel<T>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, x, mean, stddev, dy, dx, rows,
                       cols);
    return hipGetLastError();
}

#define INSTANTIATE(T)                                                                                        \
    template hipError_t launch_transpose<T>(const T*, T*, int64_t, int64_t, hipStream_t);                      \
    template hipError_t launch_layernorm_fwd<T>(const T*, T*, T*, T*, int64_t, int64_t, hipStream_t);          \
    template hipError_t launch_layernorm_bwd<T>(const T*, const T*, const T*, const T*, T*, int64_t, int64_t, hipStream_t);
INSTANTIATE(double)
INSTANTIATE(float)

}  // namespace prad
