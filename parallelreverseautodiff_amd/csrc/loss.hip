// Operations that close the loop of a training step around the matrix products, so that a whole
// forward + backward + update stays on the device: row-wise softmax
// (src/RMAD/SoftmaxOperation.cs:45-110) and the categorical cross-entropy loss
// (src/RMAD/Loss/CategoricalCrossEntropyLossOperation.cs:37-86).  They are tiny (batch x classes)
// and latency-bound: one wavefront per row, no LDS.
#include "common.h"

namespace prad {

// y[i][j] = exp(x[i][j] - max_i) / sum_j exp(x[i][j] - max_i)
template <typename T>
__global__ void __launch_bounds__(64) softmax_fwd_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t rows, int64_t cols,
                                                         T alpha) {
    const int64_t i = blockIdx.x;
    const T* __restrict__ xr = x + i * cols;
    T* __restrict__ yr = y + i * cols;
    double mx = -INFINITY;
    for (int64_t j = threadIdx.x; j < cols; j += 64) mx = fmax(mx, (double)(xr[j] * alpha));
    const T m = (T)wave_max(mx);
    double sum = 0.0;
    for (int64_t j = threadIdx.x; j < cols; j += 64) {
        const T e = dev_exp(xr[j] * alpha - m);
        yr[j] = e;
        sum += (double)e;
    }
    const T s = (T)wave_sum(sum);
    for (int64_t j = threadIdx.x; j < cols; j += 64) yr[j] = yr[j] / s;
}

// Rows of at most 64 columns (attention windows: 49): a lane holds one element of each of SHORT_ROWS consecutive
// rows, whose loads are all issued before the first reduction (a row is under 256 bytes: one row per wavefront
// leaves the memory system idle).  Each row is read once and written once.
constexpr int SHORT_ROWS = 8;
template <typename T>
__global__ void __launch_bounds__(256) softmax_fwd_short_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t rows, int64_t cols,
                                                                T alpha) {
    const int64_t i0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * SHORT_ROWS;
    const int lane = threadIdx.x & 63;
    const bool on = lane < cols;
    T xv[SHORT_ROWS];
#pragma unroll
    for (int r = 0; r < SHORT_ROWS; ++r) xv[r] = (on && i0 + r < rows) ? x[(i0 + r) * cols + lane] * alpha : (T)0;
#pragma unroll
    for (int r = 0; r < SHORT_ROWS; ++r) {
        if (i0 + r >= rows) break;
        const T m = wave_max_t(on ? xv[r] : (T)-INFINITY);
        const T e = on ? short_exp(xv[r] - m) : (T)0;
        const T s = wave_sum_t(e);
        if (on) y[(i0 + r) * cols + lane] = e / s;
    }
}
template <typename T>
__global__ void __launch_bounds__(256) softmax_bwd_short_kernel(const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dx,
                                                                int64_t rows, int64_t cols, T alpha) {
    const int64_t i0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * SHORT_ROWS;
    const int lane = threadIdx.x & 63;
    const bool on = lane < cols;
    T yv[SHORT_ROWS], gv[SHORT_ROWS];
#pragma unroll
    for (int r = 0; r < SHORT_ROWS; ++r) {
        const bool ok = on && i0 + r < rows;
        yv[r] = ok ? y[(i0 + r) * cols + lane] : (T)0;
        gv[r] = ok ? dy[(i0 + r) * cols + lane] : (T)0;
    }
#pragma unroll
    for (int r = 0; r < SHORT_ROWS; ++r) {
        if (i0 + r >= rows) break;
        const T dot = wave_sum_t(on ? gv[r] * yv[r] : (T)0);
        if (on) dx[(i0 + r) * cols + lane] = (yv[r] * (gv[r] - dot)) * alpha;
    }
}

// Many short rows (the attention scores of a windowed block: 150 528 rows of 49): a lane owns a whole row, so no
// reduction crosses lanes and the sum runs over the columns in ascending order, as the reference's does.  The
// workgroup's rows are contiguous in memory: they come in and go out as one coalesced block through LDS, where
// the odd row pitch keeps the lanes' column-by-column walk free of bank conflicts.
template <typename T> struct RowsPerGroup { static constexpr int N = 128; };
template <typename T>
__global__ void __launch_bounds__(256) softmax_fwd_rows_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t rows, int64_t cols64,
                                                               T alpha) {
    constexpr int RPG = RowsPerGroup<T>::N;
    constexpr int VEC = 16 / sizeof(T);
    constexpr int U = RPG * 64 / VEC / 256;  // 16-byte vectors per thread that cover the largest block (64 columns)
    typedef T Vec __attribute__((ext_vector_type(VEC)));
    extern __shared__ __attribute__((aligned(16))) unsigned char rows_lds[];
    T* __restrict__ tile = reinterpret_cast<T*>(rows_lds);
    const int cols = (int)cols64, pitch = cols | 1;
    const int64_t i0 = (int64_t)blockIdx.x * RPG;
    const int nrows = (int)min((int64_t)RPG, rows - i0);
    const int n = nrows * cols, nvec = n / VEC;
    const T* __restrict__ src = x + i0 * cols;   // 16-byte aligned: a block is RPG * cols elements, a multiple of 1 KiB
    T* __restrict__ dst = y + i0 * cols;
    // Element e of the block sits at row e / cols, column e % cols.  All of a thread's loads are issued before the
    // first value is parked: taken a few at a time, the block would come in as a chain of memory latencies.
    const int step = 256 * VEC, dr = step / cols, dc = step % cols;
    const int e_first = (int)threadIdx.x * VEC;
    {
        Vec tmp[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
            if ((int)threadIdx.x + 256 * u < nvec) tmp[u] = *reinterpret_cast<const Vec*>(src + e_first + step * u);
        int r = e_first / cols, c = e_first % cols;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if ((int)threadIdx.x + 256 * u < nvec) {
                int rr = r, cc = c;
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    tile[rr * pitch + cc] = tmp[u][k] * alpha;
                    if (++cc == cols) { cc = 0; ++rr; }
                }
            }
            r += dr; c += dc;
            if (c >= cols) { c -= cols; ++r; }
        }
        for (int e = nvec * VEC + threadIdx.x; e < n; e += 256) tile[(e / cols) * pitch + e % cols] = src[e] * alpha;  // ragged end
    }
    __syncthreads();
    if ((int)threadIdx.x < nrows) {
        // the row lives in registers (rows here have at most 64 columns): independent LDS reads, one pass each way
        T* __restrict__ row = tile + threadIdx.x * pitch;
        T v[64];
#pragma unroll
        for (int j = 0; j < 64; ++j) v[j] = j < cols ? row[j] : (T)-INFINITY;
        T m = v[0];
#pragma unroll
        for (int j = 1; j < 64; ++j) m = v[j] > m ? v[j] : m;
        T sum = (T)0;
#pragma unroll
        for (int j = 0; j < 64; ++j) {
            v[j] = j < cols ? short_exp(v[j] - m) : (T)0;
            sum = sum + v[j];  // columns in ascending order; the zeros past the row change nothing
        }
#pragma unroll
        for (int j = 0; j < 64; ++j)
            if (j < cols) row[j] = v[j] / sum;
    }
    __syncthreads();
    {
        int r = e_first / cols, c = e_first % cols;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if ((int)threadIdx.x + 256 * u < nvec) {
                Vec out;
                int rr = r, cc = c;
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    out[k] = tile[rr * pitch + cc];
                    if (++cc == cols) { cc = 0; ++rr; }
                }
                *reinterpret_cast<Vec*>(dst + e_first + step * u) = out;
            }
            r += dr; c += dc;
            if (c >= cols) { c -= cols; ++r; }
        }
        for (int e = nvec * VEC + threadIdx.x; e < n; e += 256) dst[e] = tile[(e / cols) * pitch + e % cols];
    }
}

// The reference multiplies dy with the explicit Jacobian row by row (O(cols^2)):
//   dx[j] = dy[j]*y[j]*(1-y[j]) - sum_{k != j} dy[k]*y[j]*y[k]  =  y[j] * (dy[j] - sum_k dy[k]*y[k]).
template <typename T>
__global__ void __launch_bounds__(64) softmax_bwd_kernel(const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dx,
                                                         int64_t rows, int64_t cols, T alpha) {
    const int64_t i = blockIdx.x;
    const T* __restrict__ yr = y + i * cols;
    const T* __restrict__ gr = dy + i * cols;
    double dot = 0.0;
    for (int64_t j = threadIdx.x; j < cols; j += 64) dot += (double)gr[j] * (double)yr[j];
    dot = wave_sum(dot);
    for (int64_t j = threadIdx.x; j < cols; j += 64) dx[i * cols + j] = (T)((double)yr[j] * ((double)gr[j] - dot)) * alpha;
}

// loss[0] = (sum_ij -t*log(p + 1e-15)) / rows ; one workgroup.
template <typename T>
__global__ void __launch_bounds__(256) cce_fwd_kernel(const T* __restrict__ p, const T* __restrict__ t, T* __restrict__ loss,
                                                      int64_t rows, int64_t cols) {
    const int64_t n = rows * cols;
    double s = 0.0;
    for (int64_t i = threadIdx.x; i < n; i += 256) {
        const T term = -t[i] * (T)log((double)(p[i] + (T)1e-15));
        s += (double)term;
    }
    s = wave_sum(s);
    __shared__ double part[4];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) loss[0] = (T)((part[0] + part[1]) + (part[2] + part[3])) / (T)rows;
}

// dp = -(1/rows) * t / (p + 1e-15)
template <typename T>
__global__ void __launch_bounds__(256) cce_bwd_kernel(const T* __restrict__ p, const T* __restrict__ t, T* __restrict__ dp,
                                                      int64_t rows, int64_t cols) {
    const int64_t n = rows * cols;
    const T scale = (T)1 / (T)rows;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
        dp[i] = -scale * t[i] / (p[i] + (T)1e-15);
}

// Softmax.Forward, CategoricalCrossEntropy.Backward and Softmax.Backward of one row by one wavefront
// (same arithmetic, statement by statement, as the three kernels above).
template <typename T>
__device__ __forceinline__ void softmax_cce_row(const T* __restrict__ xr, const T* __restrict__ tr, T* __restrict__ yr,
                                                T* __restrict__ gr, T* __restrict__ dxr, int64_t rows, int64_t cols, int lane) {
    if (cols <= 64) {  // the arithmetic of the short-row kernels, which the separate launches use for such rows
        const bool on = lane < cols;
        const T xv = on ? xr[lane] : (T)0;
        const T m = wave_max_t(on ? xv : (T)-INFINITY);
        const T e = on ? short_exp(xv - m) : (T)0;
        const T s = wave_sum_t(e);
        const T p = e / s;
        const T scale = (T)1 / (T)rows;
        const T g = on ? -scale * tr[lane] / (p + (T)1e-15) : (T)0;
        const T dot = wave_sum_t(on ? g * p : (T)0);
        if (on) { yr[lane] = p; gr[lane] = g; dxr[lane] = p * (g - dot); }
        return;
    }
    double mx = -INFINITY;
    for (int64_t j = lane; j < cols; j += 64) mx = fmax(mx, (double)xr[j]);
    const T m = (T)wave_max(mx);
    double sum = 0.0;
    for (int64_t j = lane; j < cols; j += 64) {
        const T e = dev_exp(xr[j] - m);
        yr[j] = e;
        sum += (double)e;
    }
    const T s = (T)wave_sum(sum);
    const T scale = (T)1 / (T)rows;
    double dot = 0.0;
    for (int64_t j = lane; j < cols; j += 64) {
        const T p = yr[j] / s;
        const T g = -scale * tr[j] / (p + (T)1e-15);
        yr[j] = p;
        gr[j] = g;
        dot += (double)g * (double)p;
    }
    dot = wave_sum(dot);
    for (int64_t j = lane; j < cols; j += 64) dxr[j] = (T)((double)yr[j] * ((double)gr[j] - dot));
}

// One wavefront per row, four rows per workgroup.  When the loss value is wanted, the workgroup that
// finishes last (a counter in device memory tells) forms it from the finished p exactly as cce_fwd_kernel
// does, so the whole loss stage of a step is one launch; it leaves the counter at zero for the next launch.
template <typename T>
__global__ void __launch_bounds__(256) softmax_cce_kernel(const T* __restrict__ x, const T* __restrict__ t, T* __restrict__ y,
                                                          T* __restrict__ dy, T* __restrict__ dx, T* __restrict__ loss,
                                                          unsigned* __restrict__ counter, int64_t rows, int64_t cols) {
    const int64_t i = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i < rows) {
        const int64_t o = i * cols;
        softmax_cce_row<T>(x + o, t + o, y + o, dy + o, dx + o, rows, cols, threadIdx.x & 63);
    }
    if (loss == nullptr) return;
    __shared__ int last;
    __threadfence();  // this workgroup's p is visible device-wide before its arrival is counted
    __syncthreads();
    if (threadIdx.x == 0) last = atomicAdd(counter, 1u) == gridDim.x - 1 ? 1 : 0;
    __syncthreads();
    if (!last) return;
    __threadfence();
    const volatile T* p = y;  // written by other workgroups: read past this compute unit's cache
    const int64_t n = rows * cols;
    double s = 0.0;
    for (int64_t e = threadIdx.x; e < n; e += 256) {
        const T term = -t[e] * (T)log((double)(p[e] + (T)1e-15));
        s += (double)term;
    }
    s = wave_sum(s);
    __shared__ double part[4];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        loss[0] = (T)((part[0] + part[1]) + (part[2] + part[3])) / (T)rows;
        *counter = 0u;
    }
}

// MeanSquaredErrorLossOperation (src/RMAD/Loss/MeanSquaredErrorLossOperation.cs): loss = sum (y - t)^2 / (rows*cols),
// dy = (2 / (rows*cols)) * (y - t).  The sum is taken in two levels (per workgroup, then by one thread).
// WITH_DY: the same pass also writes the gradient, value for value what mse_bwd_kernel writes.
template <typename T, bool WITH_DY>
__global__ void __launch_bounds__(256) mse_partial_kernel(const T* __restrict__ y, const T* __restrict__ t, double* __restrict__ part,
                                                          T* __restrict__ dy, int64_t n) {
    const T scale = (T)2 / (T)n;
    double s = 0.0;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        const T d = y[i] - t[i];
        s += (double)(d * d);
        if (WITH_DY) dy[i] = scale * d;
    }
    s = wave_sum(s);
    __shared__ double w[4];
    if ((threadIdx.x & 63) == 0) w[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) part[blockIdx.x] = (w[0] + w[1]) + (w[2] + w[3]);
}
// The same pass in 16-byte accesses, four vectors of each operand in flight per thread (n a multiple of the vector
// length, 16-byte aligned operands): 4-byte loads, one behind the other, left the pass at 40 % of a copy's rate.
template <typename T, bool WITH_DY>
__global__ void __launch_bounds__(256) mse_partial_vec_kernel(const T* __restrict__ y, const T* __restrict__ t, double* __restrict__ part,
                                                              T* __restrict__ dy, int64_t n) {
    constexpr int VEC = 16 / sizeof(T), FLY = 4;
    typedef T Vec __attribute__((ext_vector_type(VEC)));
    const T scale = (T)2 / (T)n;
    const int64_t nv = n / VEC, stride = (int64_t)gridDim.x * 256;
    double s = 0.0;
    for (int64_t v0 = (int64_t)blockIdx.x * 256 + threadIdx.x; v0 < nv; v0 += FLY * stride) {
        Vec a[FLY], b[FLY];
#pragma unroll
        for (int u = 0; u < FLY; ++u) {
            const int64_t v = min(v0 + u * stride, nv - 1);
            a[u] = reinterpret_cast<const Vec*>(y)[v];
            b[u] = reinterpret_cast<const Vec*>(t)[v];
        }
#pragma unroll
        for (int u = 0; u < FLY; ++u) {
            if (v0 + u * stride < nv) {
                Vec d = a[u] - b[u];
#pragma unroll
                for (int i = 0; i < VEC; ++i) s += (double)(d[i] * d[i]);
                if (WITH_DY) reinterpret_cast<Vec*>(dy)[v0 + u * stride] = d * scale;
            }
        }
    }
    s = wave_sum(s);
    __shared__ double w[4];
    if ((threadIdx.x & 63) == 0) w[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) part[blockIdx.x] = (w[0] + w[1]) + (w[2] + w[3]);
}
template <typename T>
__global__ void __launch_bounds__(64) mse_final_kernel(const double* __restrict__ part, int nparts, T* __restrict__ loss, int64_t n) {
    double s = 0.0;
    for (int i = threadIdx.x; i < nparts; i += 64) s += part[i];
    s = wave_sum(s);
    if (threadIdx.x == 0) loss[0] = (T)s / (T)n;
}
template <typename T>
__global__ void __launch_bounds__(256) mse_bwd_kernel(const T* __restrict__ y, const T* __restrict__ t, T* __restrict__ dy, int64_t n) {
    const T scale = (T)2 / (T)n;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) dy[i] = scale * (y[i] - t[i]);
}

constexpr int MSE_PARTS = 1024;
size_t mse_workspace_bytes() { return MSE_PARTS * sizeof(double); }
template <typename T>
hipError_t launch_mse_fwd(const T* y, const T* t, T* loss, double* workspace, int64_t n, hipStream_t s, T* dy) {
    int64_t blocks = (n + 255) / 256;
    if (blocks > MSE_PARTS) blocks = MSE_PARTS;
    if (blocks < 1) blocks = 1;
    const bool vec = n % (16 / sizeof(T)) == 0 && n >= 65536 && reinterpret_cast<uintptr_t>(y) % 16 == 0 && reinterpret_cast<uintptr_t>(t) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(dy) % 16 == 0;
    if (vec && dy != nullptr) hipLaunchKernelGGL((mse_partial_vec_kernel<T, true>), dim3((unsigned)blocks), dim3(256), 0, s, y, t, workspace, dy, n);
    else if (vec) hipLaunchKernelGGL((mse_partial_vec_kernel<T, false>), dim3((unsigned)blocks), dim3(256), 0, s, y, t, workspace, dy, n);
    else if (dy != nullptr) hipLaunchKernelGGL((mse_partial_kernel<T, true>), dim3((unsigned)blocks), dim3(256), 0, s, y, t, workspace, dy, n);
    else hipLaunchKernelGGL((mse_partial_kernel<T, false>), dim3((unsigned)blocks), dim3(256), 0, s, y, t, workspace, dy, n);
    hipLaunchKernelGGL((mse_final_kernel<T>), dim3(1), dim3(64), 0, s, workspace, (int)blocks, loss, n);
    return hipGetLastError();
}
template <typename T>
hipError_t launch_mse_bwd(const T* y, const T* t, T* dy, int64_t n, hipStream_t s) {
    int64_t blocks = (n + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL((mse_bwd_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, s, y, t, dy, n);
    return hipGetLastError();
}

// alpha: y = softmax(alpha * x) and dx = alpha * (J^T dy), the scaled scores of an attention block without a pass
// of their own; alpha = 1 is the plain operation (a multiplication by one changes no value).
template <typename T>
hipError_t launch_softmax_fwd(const T* x, T* y, int64_t rows, int64_t cols, T alpha, hipStream_t s) {
    if (rows <= 0 || cols <= 0) return hipSuccess;
    constexpr int RPG = RowsPerGroup<T>::N;
    const bool aligned = reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0;
    if (cols <= 64 && rows >= 16 * RPG && aligned) {  // enough rows to fill the chip a lane per row
        const size_t lds = (size_t)RPG * ((size_t)cols | 1) * sizeof(T);
        hipLaunchKernelGGL((softmax_fwd_rows_kernel<T>), dim3((unsigned)((rows + RPG - 1) / RPG)), dim3(256), lds, s, x, y, rows, cols, alpha);
        return hipGetLastError();
    }
    if (cols <= 64) {
        hipLaunchKernelGGL((softmax_fwd_short_kernel<T>), dim3((unsigned)((rows + 4 * SHORT_ROWS - 1) / (4 * SHORT_ROWS))), dim3(256), 0, s, x, y,
                           rows, cols, alpha);
        return hipGetLastError();
    }
    hipLaunchKernelGGL((softmax_fwd_kernel<T>), dim3((unsigned)rows), dim3(64), 0, s, x, y, rows, cols, alpha);
    return hipGetLastError();
}
template <typename T>
hipError_t launch_softmax_bwd(const T* y, const T* dy, T* dx, int64_t rows, int64_t cols, T alpha, hipStream_t s) {
    if (rows <= 0) return hipSuccess;
    if (cols <= 64) {
        hipLaunchKernelGGL((softmax_bwd_short_kernel<T>), dim3((unsigned)((rows + 4 * SHORT_ROWS - 1) / (4 * SHORT_ROWS))), dim3(256), 0, s, y, dy,
                           dx, rows, cols, alpha);
        return hipGetLastError();
    }
    hipLaunchKernelGGL((softmax_bwd_kernel<T>), dim3((unsigned)rows), dim3(64), 0, s, y, dy, dx, rows, cols, alpha);
    return hipGetLastError();
}
// counter: one unsigned in device memory that is zero between launches (not shared with a launch that may
// run at the same time).
template <typename T>
hipError_t launch_softmax_cce(const T* x, const T* t, T* y, T* dy, T* dx, T* loss, unsigned* counter, int64_t rows, int64_t cols,
                              hipStream_t s) {
    if (rows <= 0) return hipSuccess;
    hipLaunchKernelGGL((softmax_cce_kernel<T>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, x, t, y, dy, dx, loss, counter, rows,
                       cols);
    return hipGetLastError();
}
template <typename T>
hipError_t launch_cce_fwd(const T* p, const T* t, T* loss, int64_t rows, int64_t cols, hipStream_t s) {
    hipLaunchKernelGGL((cce_fwd_kernel<T>), dim3(1), dim3(256), 0, s, p, t, loss, rows, cols);
    return hipGetLastError();
}
template <typename T>
hipError_t launch_cce_bwd(const T* p, const T* t, T* dp, int64_t rows, int64_t cols, hipStream_t s) {
    int64_t blocks = (rows * cols + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL((cce_bwd_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, s, p, t, dp, rows, cols);
    return hipGetLastError();
}

#define INSTANTIATE(T)                                                                              \
    template hipError_t launch_softmax_fwd<T>(const T*, T*, int64_t, int64_t, T, hipStream_t);         \
    template hipError_t launch_softmax_bwd<T>(const T*, const T*, T*, int64_t, int64_t, T, hipStream_t); \
    template hipError_t launch_softmax_cce<T>(const T*, const T*, T*, T*, T*, T*, unsigned*, int64_t, int64_t, hipStream_t); \
    template hipError_t launch_cce_fwd<T>(const T*, const T*, T*, int64_t, int64_t, hipStream_t);   \
    template hipError_t launch_cce_bwd<T>(const T*, const T*, T*, int64_t, int64_t, hipStream_t);   \
    template hipError_t launch_mse_fwd<T>(const T*, const T*, T*, double*, int64_t, hipStream_t, T*);   \
    template hipError_t launch_mse_bwd<T>(const T*, const T*, T*, int64_t, hipStream_t);
INSTANTIATE(double)
INSTANTIATE(float)

}  // namespace prad
