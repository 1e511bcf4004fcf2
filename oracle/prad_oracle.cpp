// TEST INFRASTRUCTURE ONLY -- NOT PART OF THE SHIPPED LIBRARY.
//
// CPU restatement of ParallelReverseAutoDiff's matrix-multiply forward/backward path and
// the gradient kernels around it.  It exists so the HIP kernels can be checked against the
// reference's arithmetic, and so the benchmark can time the reference's CPU algorithm on the
// host cores.  Only tests, the smoke check and the benchmark's cpu_baseline leg may load it;
// the product library never links or calls anything in this file.
//
// Arithmetic model: the reference is C# compiled by RyuJIT for x64, which evaluates every
// double/float multiply and add as one scalar SSE2 operation rounded to its own type and never
// contracts a*b+c into an FMA.  This file is therefore built with -O2 -ffp-contract=off and no
// fast-math, and follows the reference loop by loop (same loop order, same accumulator
// variable, same association of every expression).  T = double restates PRAD, T = float
// restates PRADLite (whose sources are the same text with double replaced by float).
//
// Storage: the reference Matrix is jagged (one array per row, src/RMAD/Matrix.cs:43-55).
// Every routine here walks rows through an array of row pointers; the entry points that take a
// contiguous buffer only build that pointer array over it, the timing entry point allocates
// each row separately like the reference does.
//
// Pinning status of each function (what independent fact checks it) is listed in
// tests/test_oracle.py next to the test that does it (the loss functions and the whole-step
// compositions of oracle/compose.py: tests/test_oracle_compose.py); functions whose libm calls (exp, tanh,
// pow) may differ from .NET's in the last ulp say so below.

#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <chrono>
#include <thread>
#include <vector>
#include <algorithm>

namespace {

// Static row partition over `threads` workers: the stand-in for Parallel.For(0, rows, i => ...)
// (src/RMAD/MatrixMultiplyOperation.cs:67,94,110).  Rows are independent, so the partition
// does not change any result.
template <class F>
void parallel_rows(int rows, int threads, F body) {
    if (threads <= 1 || rows <= 1) {
        for (int i = 0; i < rows; ++i) body(i);
        return;
    }
    threads = std::min(threads, rows);
    std::vector<std::thread> pool;
    pool.reserve(threads);
    for (int t = 0; t < threads; ++t) {
        int lo = (int)((int64_t)rows * t / threads);
        int hi = (int)((int64_t)rows * (t + 1) / threads);
        pool.emplace_back([=]() { for (int i = lo; i < hi; ++i) body(i); });
    }
    for (auto& th : pool) th.join();
}

template <class T>
std::vector<T*> row_ptrs(T* base, int rows, int64_t ld) {
    std::vector<T*> r((size_t)rows);
    for (int i = 0; i < rows; ++i) r[i] = base + (int64_t)i * ld;
    return r;
}

// ---------------------------------------------------------------------------------------
// MatrixMultiplyOperation  (src/RMAD/MatrixMultiplyOperation.cs)
// ---------------------------------------------------------------------------------------

// Forward, :67-77.  C[i][j] is zeroed and then accumulated through memory, k ascending.
template <class T>
void matmul_fwd(const T* const* A, const T* const* B, T* const* C, int M, int K, int N, int threads) {
    parallel_rows(M, threads, [=](int i) {
        for (int j = 0; j < N; ++j) {
            C[i][j] = 0;
            for (int k = 0; k < K; ++k) {
                C[i][j] += A[i][k] * B[k][j];
            }
        }
    });
}

// Backward, :94-104 (dInput1) and :110-120 (dInput2).  A is M x K, B is K x N, dC is M x N.
template <class T>
void matmul_bwd(const T* const* dC, const T* const* A, const T* const* B, T* const* dA, T* const* dB,
                int M, int K, int N, int threads) {
    parallel_rows(M, threads, [=](int i) {
        for (int j = 0; j < K; ++j) {
            dA[i][j] = 0;
            for (int k = 0; k < N; ++k) {
                dA[i][j] += dC[i][k] * B[j][k];
            }
        }
    });
    parallel_rows(K, threads, [=](int i) {
        for (int j = 0; j < N; ++j) {
            dB[i][j] = 0;
            for (int k = 0; k < M; ++k) {
                dB[i][j] += A[k][i] * dC[k][j];
            }
        }
    });
}

// The ILGPU kernel's summation order (src/RMAD/GpuMatrixMultiplyOperation.cs:51-90): the
// reduction is cut into tiles of 8, each tile's products are summed into `sum` (k ascending,
// zero padding past K), then `total += sum`.
template <class T>
void matmul_fwd_tiled8(const T* const* A, const T* const* B, T* const* C, int M, int K, int N, int threads) {
    parallel_rows(M, threads, [=](int i) {
        for (int j = 0; j < N; ++j) {
            T total = 0;
            for (int k0 = 0; k0 < K; k0 += 8) {
                T sum = 0;
                for (int k = k0; k < k0 + 8; ++k) {
                    T a = k < K ? A[i][k] : (T)0;
                    T b = k < K ? B[k][j] : (T)0;
                    sum += a * b;
                }
                total += sum;
            }
            C[i][j] = total;
        }
    });
}

// ---------------------------------------------------------------------------------------
// MatrixMultiplyAndSumOperation (src/RMAD/MatrixMultiplyAndSumOperation.cs:50-89), with
// Matrix.operator* (src/RMAD/Matrix.cs:297-326: local `sum`, k ascending), Matrix.Sum()
// (:588-606: per-row sums, then LINQ Sum over the row sums), operator*(Matrix, scalar)
// (:334-350) and Transpose (:551-566).
// ---------------------------------------------------------------------------------------

// LINQ Enumerable.Sum: over double[] it adds in double; over float[] it also accumulates in a
// double and casts the total to float once.
inline double linq_sum(const double* v, int n) { double s = 0; for (int i = 0; i < n; ++i) s += v[i]; return s; }
inline float linq_sum(const float* v, int n) { double s = 0; for (int i = 0; i < n; ++i) s += (double)v[i]; return (float)s; }

template <class T>
void matmul_sum_fwd(const T* const* A, const T* const* const* B, T* out, int M, int K, int N, int P, int threads) {
    std::vector<T> prod((size_t)M * N);
    std::vector<T> rowSums((size_t)M);
    for (int q = 0; q < P; ++q) {
        const T* const* Bq = B[q];
        T* prodp = prod.data();
        parallel_rows(M, threads, [=](int i) {
            for (int j = 0; j < N; ++j) {
                T sum = 0;
                for (int k = 0; k < K; ++k) sum += A[i][k] * Bq[k][j];
                prodp[(size_t)i * N + j] = sum;
            }
        });
        for (int i = 0; i < M; ++i) {
            T localRowSum = 0;
            for (int j = 0; j < N; ++j) localRowSum += prodp[(size_t)i * N + j];
            rowSums[i] = localRowSum;
        }
        out[q] = linq_sum(rowSums.data(), M);
    }
}

// Backward as written (:70-89): dB[q] = transpose(A) * dOut[q]  (K x M),
// dA = sum_q transpose(B[q]) * dOut[q]  (N x K, stored into an M x K matrix: needs N==M... the
// reference's operator+ walks dA's shape, so the caller guarantees (N x K) == (M x K)).
// dA starts as zeros and is re-created by operator+ each q: dA[i][j] = dA[i][j] + t[i][j].
template <class T>
void matmul_sum_bwd(const T* const* A, const T* const* const* B, const T* dOut,
                    T* const* dA, T* const* const* dB, int M, int K, int N, int P) {
    for (int i = 0; i < M; ++i) for (int j = 0; j < K; ++j) dA[i][j] = 0;
    for (int q = 0; q < P; ++q) {
        T s = dOut[q];
        for (int i = 0; i < K; ++i)
            for (int j = 0; j < M; ++j) dB[q][i][j] = A[j][i] * s;
        for (int i = 0; i < M; ++i)
            for (int j = 0; j < K; ++j) dA[i][j] = dA[i][j] + (B[q][j][i] * s);
    }
}

// ---------------------------------------------------------------------------------------
// Elementwise operations.  PradMath (src/PRAD/PradMath.cs:122-215): the double overloads are
// Math.X; the float overloads are (float)Math.X((double)x).  libm's exp/tanh/pow stand in for
// .NET's (which forwards to the platform C runtime): last-ulp agreement is not guaranteed.
// ---------------------------------------------------------------------------------------

inline double p_exp(double x) { return std::exp(x); }
inline float p_exp(float x) { return (float)std::exp((double)x); }
inline double p_tanh(double x) { return std::tanh(x); }
inline float p_tanh(float x) { return (float)std::tanh((double)x); }
inline double p_pow(double x, double y) { return std::pow(x, y); }
inline float p_pow(float x, float y) { return (float)std::pow((double)x, (double)y); }
inline double p_sqrt(double x) { return std::sqrt(x); }
inline float p_sqrt(float x) { return (float)std::sqrt((double)x); }

// LeakyReLUOperation (src/RMAD/LeakyReLUOperation.cs:54-71, 74-93).
template <class T> void leakyrelu_fwd(const T* x, T* y, int64_t n, T alpha) {
    for (int64_t i = 0; i < n; ++i) y[i] = x[i] > 0 ? x[i] : alpha * x[i];
}
template <class T> void leakyrelu_bwd(const T* x, const T* dy, T* dx, int64_t n, T alpha) {
    for (int64_t i = 0; i < n; ++i) { T g = x[i] > 0 ? (T)1.0 : alpha; dx[i] = dy[i] * g; }
}

// SigmoidOperation (src/RMAD/SigmoidOperation.cs:46-62, 65-84); backward uses the cached output.
template <class T> void sigmoid_fwd(const T* x, T* y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = (T)1.0f / ((T)1.0f + p_exp(-x[i]));
}
template <class T> void sigmoid_bwd(const T* y, const T* dy, T* dx, int64_t n) {
    for (int64_t i = 0; i < n; ++i) { T d = y[i] * (1 - y[i]); dx[i] = dy[i] * d; }
}

// TanhOperation (src/RMAD/TanhOperation.cs:42-57, 60-79).
template <class T> void tanh_fwd(const T* x, T* y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = p_tanh(x[i]);
}
template <class T> void tanh_bwd(const T* y, const T* dy, T* dx, int64_t n) {
    for (int64_t i = 0; i < n; ++i) { T d = 1 - p_pow(y[i], (T)2); dx[i] = dy[i] * d; }
}

// GELUOperation (src/RMAD/GELUOperation.cs:86-101; float twin
// lite/src/ParallelReverseAutoDiffLite/Lite/GELUOperation.cs:86-100).  The backward formula is
// the reference's own (squared sech^2 term and an extra 0.5*x*b), not the analytic derivative.
inline double gelu_s(double) { return p_sqrt(2 / M_PI); }
inline float gelu_s(float) { const float pi = (float)M_PI; return p_sqrt(2 / pi); }
template <class T> inline T gelu_c0();
template <> inline double gelu_c0<double>() { return 0.044715; }
template <> inline float gelu_c0<float>() { return 0.044715f; }

template <class T> void gelu_fwd(const T* x, T* y, int64_t n) {
    const T s = gelu_s((T)0), c0 = gelu_c0<T>();
    for (int64_t i = 0; i < n; ++i) {
        T xi = x[i];
        T a = (T)0.5 * ((T)1.0 + p_tanh(s * (xi + (c0 * p_pow(xi, (T)3)))));
        y[i] = a * xi;
    }
}
template <class T> void gelu_bwd(const T* x, const T* dy, T* dx, int64_t n) {
    const T s = gelu_s((T)0), c0 = gelu_c0<T>();
    for (int64_t i = 0; i < n; ++i) {
        T xi = x[i];
        T b = p_tanh(s * (xi + (c0 * p_pow(xi, (T)3))));
        T c = p_pow(1 - p_pow(b, (T)2), (T)2);
        T d = s * ((c0 * 3 * p_pow(xi, (T)2)) + 1);
        T g = ((T)0.5 * xi * ((c * d) + b)) + ((T)0.5 * (1 + b));
        dx[i] = dy[i] * g;
    }
}

// HadamardProductOperation (src/RMAD/HadamardProductOperation.cs:50-81, 84-118).
template <class T> void hadamard_fwd(const T* a, const T* b, T* y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = a[i] * b[i];
}
template <class T> void hadamard_bwd(const T* a, const T* b, const T* dy, T* da, T* db, int64_t n) {
    for (int64_t i = 0; i < n; ++i) { da[i] = dy[i] * b[i]; db[i] = dy[i] * a[i]; }
}

// OperationBase.AccumulateGradient (src/RMAD/OperationBase.cs:295-303): dest += grad.
template <class T> void accumulate(T* dest, const T* grad, int64_t n) {
    for (int64_t i = 0; i < n; ++i) dest[i] += grad[i];
}

// ---------------------------------------------------------------------------------------
// GradientClipper.ClipGradients + StandardizedMatrix (src/RMAD/GradientClipper.cs:118-157,
// 212-253; float twin lite/.../GradientClipper.cs keeps sum/mean/variance in float).
// ---------------------------------------------------------------------------------------

// .NET Math.Min returns NaN when either argument is NaN (C fmin would return the other one).
template <class T> inline T dotnet_min(T a, T b) {
    if (a != a) return a;
    if (b != b) return b;
    return a < b ? a : b;
}

template <class T> void clip_gradients(T* g, int64_t n, T clipValue, T minValue) {
    T sum = 0;
    int64_t count = 0;
    for (int64_t i = 0; i < n; ++i) { sum += g[i]; count++; }
    T mean = sum / count;
    T varianceSum = 0;
    for (int64_t i = 0; i < n; ++i) varianceSum += p_pow(g[i] - mean, (T)2);
    T stdDev = p_sqrt(varianceSum / count);
    for (int64_t i = 0; i < n; ++i) {
        T z = (g[i] - mean) / stdDev;
        T value = dotnet_min(clipValue, 1 + std::fabs(z));
        if (g[i] > value) g[i] = value;
        else if (g[i] < -value) g[i] = -value;
        if (g[i] > 0 && g[i] < minValue) g[i] = minValue;
        else if (g[i] < 0 && g[i] > -minValue) g[i] = -minValue;
    }
}

// ---------------------------------------------------------------------------------------
// AdamOptimizer.UpdateWeightWithAdam (src/RMAD/AdamOptimizer.cs:195-239) with the helpers in
// src/RMAD/MatrixUtils.cs:71-139; ReverseAdamUpdate (:158-193) is its algebraic inverse.
// ---------------------------------------------------------------------------------------
template <class T> void adam_update(T* w, T* m, T* v, const T* g, int64_t n, T lr, T beta1, T beta2, T eps, T t) {
    const T c1 = 1 / (1 - p_pow(beta1, t));
    const T c2 = 1 / (1 - p_pow(beta2, t));
    const T omb1 = 1 - beta1, omb2 = 1 - beta2;
    for (int64_t i = 0; i < n; ++i) {
        T firstMoment = (beta1 * m[i]) + (omb1 * g[i]);
        T secondMoment = (beta2 * v[i]) + (omb2 * (g[i] * g[i]));
        T mhat = c1 * firstMoment;
        T vhat = c2 * secondMoment;
        T red = lr * mhat / (p_sqrt(vhat) + eps);
        w[i] -= red;
        m[i] = firstMoment;
        v[i] = secondMoment;
    }
}
template <class T> void adam_reverse(T* w, T* m, T* v, const T* g, int64_t n, T lr, T beta1, T beta2, T eps, T t) {
    const T c1 = 1 / (1 - p_pow(beta1, t));
    const T c2 = 1 / (1 - p_pow(beta2, t));
    for (int64_t i = 0; i < n; ++i) {
        T mhat = c1 * m[i];
        T vhat = c2 * v[i];
        T red = lr * mhat / (p_sqrt(vhat) + eps);
        w[i] += red;
    }
    for (int64_t i = 0; i < n; ++i) m[i] = (m[i] - ((1 - beta1) * g[i])) / beta1;
    for (int64_t i = 0; i < n; ++i) v[i] = (v[i] - ((1 - beta2) * g[i] * g[i])) / beta2;
}

// ---------------------------------------------------------------------------------------
// Ops next to the matmuls in the MLP configuration (restated only to compose a training step).
// ---------------------------------------------------------------------------------------

// MatrixAddBroadcastingOperation (src/RMAD/MatrixAddBroadcastingOperation.cs:32-70):
// y[i][j] = x[i][j] + b[0][j]; backward passes dy through and db[0][j] = sum_i dy[i][j]
// (Column(j).Sum(): LINQ sum over the column, rows ascending).
template <class T> void add_broadcast_fwd(const T* x, const T* b, T* y, int rows, int cols) {
    for (int i = 0; i < rows; ++i) for (int j = 0; j < cols; ++j) y[(size_t)i * cols + j] = x[(size_t)i * cols + j] + b[j];
}
template <class T> void add_broadcast_bwd_bias(const T* dy, T* db, int rows, int cols) {
    std::vector<T> col((size_t)rows);
    for (int j = 0; j < cols; ++j) {
        for (int i = 0; i < rows; ++i) col[i] = dy[(size_t)i * cols + j];
        db[j] = linq_sum(col.data(), rows);
    }
}

// SoftmaxOperation (src/RMAD/SoftmaxOperation.cs:45-110): row-wise, subtract the row maximum,
// exponentiate, divide by the sum; backward is the explicit Jacobian product per row:
// sum += dy[k]*y[j]*(1-y[j]) for k==j, sum -= dy[k]*y[j]*y[k] otherwise (products left to right).
template <class T> void softmax_fwd(const T* x, T* y, int rows, int cols) {
    for (int i = 0; i < rows; ++i) {
        const T* xr = x + (size_t)i * cols; T* yr = y + (size_t)i * cols;
        T mx = xr[0];
        for (int j = 1; j < cols; ++j) if (xr[j] > mx) mx = xr[j];
        T sum = 0;
        for (int j = 0; j < cols; ++j) { yr[j] = p_exp(xr[j] - mx); sum += yr[j]; }
        for (int j = 0; j < cols; ++j) yr[j] = yr[j] / sum;
    }
}
template <class T> void softmax_bwd(const T* y, const T* dy, T* dx, int rows, int cols) {
    for (int i = 0; i < rows; ++i) {
        const T* yr = y + (size_t)i * cols; const T* gr = dy + (size_t)i * cols; T* dr = dx + (size_t)i * cols;
        for (int j = 0; j < cols; ++j) {
            T acc = 0;
            for (int k = 0; k < cols; ++k) {
                if (j == k) acc += gr[k] * yr[j] * (1 - yr[j]);
                else acc -= gr[k] * yr[j] * yr[k];
            }
            dr[j] = acc;
        }
    }
}

// CategoricalCrossEntropyLossOperation (src/RMAD/Loss/CategoricalCrossEntropyLossOperation.cs:37-86):
// loss = (LINQ sum over ij of -t*log(p + 1e-15)) / rows ; dp = -(1/rows) * t / (p + 1e-15).
template <class T> T cce_fwd(const T* p, const T* t, int rows, int cols) {
    std::vector<T> terms((size_t)rows * cols);
    for (size_t i = 0; i < terms.size(); ++i) terms[i] = -t[i] * (T)std::log((double)(p[i] + (T)1e-15));
    return linq_sum(terms.data(), (int)terms.size()) / rows;
}
template <class T> void cce_bwd(const T* p, const T* t, T* dp, int rows, int cols) {
    for (int64_t i = 0; i < (int64_t)rows * cols; ++i) dp[i] = -((T)1.0 / rows) * t[i] / (p[i] + (T)1e-15);
}

// MeanSquaredErrorLossOperation (src/RMAD/Loss/MeanSquaredErrorLossOperation.cs): LINQ sum of diff*diff over all
// elements, divided by rows*cols; gradient (2/(rows*cols)) * (y - t).
template <class T> T mse_fwd(const T* y, const T* t, int rows, int cols) {
    std::vector<T> terms((size_t)rows * cols);
    for (size_t i = 0; i < terms.size(); ++i) { T d = y[i] - t[i]; terms[i] = d * d; }
    return linq_sum(terms.data(), (int)terms.size()) / (rows * cols);
}
template <class T> void mse_bwd(const T* y, const T* t, T* dy, int rows, int cols) {
    const T scale = (T)2 / (rows * cols);
    for (int64_t i = 0; i < (int64_t)rows * cols; ++i) dy[i] = scale * (y[i] - t[i]);
}

// ---------------------------------------------------------------------------------------
// Operations adjacent to the products in the reference's example graphs.
// ---------------------------------------------------------------------------------------

// MatrixAddOperation (src/RMAD/MatrixAddOperation.cs:30-68): y = a + b; both input gradients are copies of dy.
template <class T> void matrix_add(const T* a, const T* b, T* y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = a[i] + b[i];
}
// MatrixAddThreeOperation (src/RMAD/MatrixAddThreeOperation.cs:35-70): y = a + b + bias, left to right.
template <class T> void matrix_add_three(const T* a, const T* b, const T* c, T* y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = a[i] + b[i] + c[i];
}
// MatrixTransposeOperation (src/RMAD/MatrixTransposeOperation.cs:30-64): y[i][j] = x[j][i]; backward transposes dy.
template <class T> void matrix_transpose(const T* x, T* y, int rows, int cols) {
    for (int i = 0; i < cols; ++i) for (int j = 0; j < rows; ++j) y[(size_t)i * rows + j] = x[(size_t)j * cols + i];
}

// LINQ Average: double[] sums in double and divides by the count; float[] sums in double and
// returns (float)(sum / count).
inline double linq_average(const double* x, int n) { double s = 0; for (int i = 0; i < n; ++i) s += x[i]; return s / n; }
inline float linq_average(const float* x, int n) { double s = 0; for (int i = 0; i < n; ++i) s += (double)x[i]; return (float)(s / n); }

// LayerNormalizationOperation (src/RMAD/LayerNormalizationOperation.cs:56-110, EPSILON = 1e-9 :17):
// per row mean = Average(), stdDev = sqrt(Sum(pow(x - mean, 2)) / cols), y = (x - mean) / (stdDev + eps).
// Backward AS WRITTEN (:87-110): dx = dy * ((1 - 1/cols) / (stdDev + eps) - (x - mean)^2 / (cols * (stdDev + eps)^3)),
// the diagonal of the Jacobian only (not the full layer-norm gradient).
template <class T> void layernorm_fwd(const T* x, T* y, T* mean, T* stddev, int rows, int cols) {
    const T eps = (T)1e-9;
    std::vector<T> sq((size_t)cols);
    for (int i = 0; i < rows; ++i) {
        const T* xr = x + (size_t)i * cols;
        mean[i] = linq_average(xr, cols);
        for (int j = 0; j < cols; ++j) sq[j] = p_pow(xr[j] - mean[i], (T)2);
        stddev[i] = (T)std::sqrt((double)(linq_sum(sq.data(), cols) / cols));
        for (int j = 0; j < cols; ++j) y[(size_t)i * cols + j] = (xr[j] - mean[i]) / (stddev[i] + eps);
    }
}
template <class T> void layernorm_bwd(const T* x, const T* mean, const T* stddev, const T* dy, T* dx, int rows, int cols) {
    const T eps = (T)1e-9;
    for (int i = 0; i < rows; ++i) {
        const T inv = 1 / (stddev[i] + eps);
        const T exp1 = (1 - ((T)1.0 / cols)) * inv;
        for (int j = 0; j < cols; ++j) {
            const size_t e = (size_t)i * cols + j;
            const T exp2 = p_pow(x[e] - mean[i], (T)2) / (cols * p_pow(stddev[i] + eps, (T)3));
            dx[e] = dy[e] * (exp1 - exp2);
        }
    }
}

// AmplifiedSigmoidOperation (src/RMAD/AmplifiedSigmoidOperation.cs:44-84): y = 1 / (1 + pow(PI - 2, -x)) where
// PradMath.PI is a float ((float)Math.PI, src/PRAD/PradMath.cs:20) and PI - 2 a float subtraction, widened to
// double for Math.Pow in the double build.  Backward AS WRITTEN: dx = dy * pow(b, -x) / pow(1 + pow(b, -x), 2)
// (without the ln(b) factor of the derivative).  PRADLite has no such operation; the float instantiation
// follows the same text with PradMath.Pow(float, float) = (float)Math.Pow.
template <class T> inline T amp_base() { return (T)((float)3.14159265358979323846 - 2.0f); }
template <class T> void amplified_sigmoid_fwd(const T* x, T* y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = (T)1 / ((T)1 + p_pow(amp_base<T>(), -x[i]));
}
template <class T> void amplified_sigmoid_bwd(const T* x, const T* dy, T* dx, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        const T d = p_pow(amp_base<T>(), -x[i]) / p_pow((T)1 + p_pow(amp_base<T>(), -x[i]), (T)2);
        dx[i] = dy[i] * d;
    }
}

// ---------------------------------------------------------------------------------------
// Seeded fill used only by the timing entry point: SplitMix64 of (seed, tensor, index).
// ---------------------------------------------------------------------------------------
inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
inline double u01(uint64_t seed, uint64_t tensor, uint64_t idx) {
    uint64_t z = splitmix64(splitmix64(seed ^ (tensor * 0xD1B54A32D192ED03ull)) + idx);
    return (double)(z >> 11) * (1.0 / 9007199254740992.0);
}

template <class T>
struct Jagged {
    int rows, cols;
    std::vector<T*> r;
    Jagged(int rows_, int cols_) : rows(rows_), cols(cols_), r((size_t)rows_) {
        for (int i = 0; i < rows; ++i) r[i] = (T*)std::calloc((size_t)cols, sizeof(T));  // one allocation per row
    }
    ~Jagged() { for (T* p : r) std::free(p); }
    void fill(uint64_t seed, uint64_t tensor, double lo, double hi) {
        for (int i = 0; i < rows; ++i) for (int j = 0; j < cols; ++j)
            r[i][j] = (T)(lo + (hi - lo) * u01(seed, tensor, (uint64_t)i * cols + j));
    }
};

// Times `iters` forward+backward passes of an N x N x N product on separately allocated rows.
template <class T>
double time_matmul_fwdbwd(int N, int threads, int iters, double* checksum) {
    Jagged<T> A(N, N), B(N, N), dC(N, N), C(N, N), dA(N, N), dB(N, N);
    A.fill(20240611, 1, -1, 1); B.fill(20240611, 2, -1, 1); dC.fill(20240611, 3, -1, 1);
    auto t0 = std::chrono::steady_clock::now();
    for (int it = 0; it < iters; ++it) {
        matmul_fwd<T>(A.r.data(), B.r.data(), C.r.data(), N, N, N, threads);
        matmul_bwd<T>(dC.r.data(), A.r.data(), B.r.data(), dA.r.data(), dB.r.data(), N, N, N, threads);
    }
    auto t1 = std::chrono::steady_clock::now();
    if (checksum) *checksum = (double)C.r[N / 2][N / 3] + (double)dA.r[N / 3][N / 2] + (double)dB.r[N - 1][0];
    return std::chrono::duration<double>(t1 - t0).count();
}

}  // namespace

// ---------------------------------------------------------------------------------------
// C entry points (contiguous row-major buffers with a leading dimension equal to the column
// count; the row-pointer arrays are built here).
// ---------------------------------------------------------------------------------------
#define EXPORT extern "C" __attribute__((visibility("default")))

#define DEFINE_ENTRY_POINTS(SFX, T)                                                                            \
    EXPORT void oracle_matmul_fwd_##SFX(const T* A, const T* B, T* C, int M, int K, int N, int threads) {      \
        auto a = row_ptrs<const T>(A, M, K); auto b = row_ptrs<const T>(B, K, N); auto c = row_ptrs<T>(C, M, N); \
        matmul_fwd<T>(a.data(), b.data(), c.data(), M, K, N, threads);                                         \
    }                                                                                                          \
    EXPORT void oracle_matmul_fwd_tiled8_##SFX(const T* A, const T* B, T* C, int M, int K, int N, int threads) { \
        auto a = row_ptrs<const T>(A, M, K); auto b = row_ptrs<const T>(B, K, N); auto c = row_ptrs<T>(C, M, N); \
        matmul_fwd_tiled8<T>(a.data(), b.data(), c.data(), M, K, N, threads);                                  \
    }                                                                                                          \
    EXPORT void oracle_matmul_bwd_##SFX(const T* dC, const T* A, const T* B, T* dA, T* dB, int M, int K, int N, \
                                        int threads) {                                                         \
        auto g = row_ptrs<const T>(dC, M, N); auto a = row_ptrs<const T>(A, M, K);                             \
        auto b = row_ptrs<const T>(B, K, N); auto da = row_ptrs<T>(dA, M, K); auto db = row_ptrs<T>(dB, K, N); \
        matmul_bwd<T>(g.data(), a.data(), b.data(), da.data(), db.data(), M, K, N, threads);                   \
    }                                                                                                          \
    EXPORT void oracle_matmul_sum_fwd_##SFX(const T* A, const T* B, T* out, int M, int K, int N, int P,        \
                                            int threads) {                                                     \
        auto a = row_ptrs<const T>(A, M, K);                                                                   \
        std::vector<std::vector<const T*>> bq; std::vector<const T* const*> bp;                                \
        for (int q = 0; q < P; ++q) bq.push_back(row_ptrs<const T>(B + (size_t)q * K * N, K, N));              \
        for (int q = 0; q < P; ++q) bp.push_back(bq[q].data());                                                \
        matmul_sum_fwd<T>(a.data(), bp.data(), out, M, K, N, P, threads);                                      \
    }                                                                                                          \
    EXPORT void oracle_matmul_sum_bwd_##SFX(const T* A, const T* B, const T* dOut, T* dA, T* dB, int M, int K, \
                                            int N, int P) {                                                    \
        auto a = row_ptrs<const T>(A, M, K); auto da = row_ptrs<T>(dA, M, K);                                  \
        std::vector<std::vector<const T*>> bq; std::vector<const T* const*> bp;                                \
        std::vector<std::vector<T*>> dq; std::vector<T* const*> dp;                                            \
        for (int q = 0; q < P; ++q) bq.push_back(row_ptrs<const T>(B + (size_t)q * K * N, K, N));              \
        for (int q = 0; q < P; ++q) dq.push_back(row_ptrs<T>(dB + (size_t)q * K * M, K, M));                   \
        for (int q = 0; q < P; ++q) { bp.push_back(bq[q].data()); dp.push_back(dq[q].data()); }                \
        matmul_sum_bwd<T>(a.data(), bp.data(), dOut, da.data(), dp.data(), M, K, N, P);                        \
    }                                                                                                          \
    EXPORT void oracle_leakyrelu_fwd_##SFX(const T* x, T* y, int64_t n, T alpha) { leakyrelu_fwd<T>(x, y, n, alpha); } \
    EXPORT void oracle_leakyrelu_bwd_##SFX(const T* x, const T* dy, T* dx, int64_t n, T alpha) {               \
        leakyrelu_bwd<T>(x, dy, dx, n, alpha);                                                                 \
    }                                                                                                          \
    EXPORT void oracle_sigmoid_fwd_##SFX(const T* x, T* y, int64_t n) { sigmoid_fwd<T>(x, y, n); }             \
    EXPORT void oracle_sigmoid_bwd_##SFX(const T* y, const T* dy, T* dx, int64_t n) { sigmoid_bwd<T>(y, dy, dx, n); } \
    EXPORT void oracle_tanh_fwd_##SFX(const T* x, T* y, int64_t n) { tanh_fwd<T>(x, y, n); }                   \
    EXPORT void oracle_tanh_bwd_##SFX(const T* y, const T* dy, T* dx, int64_t n) { tanh_bwd<T>(y, dy, dx, n); } \
    EXPORT void oracle_gelu_fwd_##SFX(const T* x, T* y, int64_t n) { gelu_fwd<T>(x, y, n); }                   \
    EXPORT void oracle_gelu_bwd_##SFX(const T* x, const T* dy, T* dx, int64_t n) { gelu_bwd<T>(x, dy, dx, n); } \
    EXPORT void oracle_hadamard_fwd_##SFX(const T* a, const T* b, T* y, int64_t n) { hadamard_fwd<T>(a, b, y, n); } \
    EXPORT void oracle_hadamard_bwd_##SFX(const T* a, const T* b, const T* dy, T* da, T* db, int64_t n) {      \
        hadamard_bwd<T>(a, b, dy, da, db, n);                                                                  \
    }                                                                                                          \
    EXPORT void oracle_accumulate_##SFX(T* dest, const T* grad, int64_t n) { accumulate<T>(dest, grad, n); }   \
    EXPORT void oracle_clip_##SFX(T* g, int64_t n, T clipValue, T minValue) { clip_gradients<T>(g, n, clipValue, minValue); } \
    EXPORT void oracle_adam_##SFX(T* w, T* m, T* v, const T* g, int64_t n, T lr, T b1, T b2, T eps, T t) {     \
        adam_update<T>(w, m, v, g, n, lr, b1, b2, eps, t);                                                     \
    }                                                                                                          \
    EXPORT void oracle_adam_reverse_##SFX(T* w, T* m, T* v, const T* g, int64_t n, T lr, T b1, T b2, T eps, T t) { \
        adam_reverse<T>(w, m, v, g, n, lr, b1, b2, eps, t);                                                    \
    }                                                                                                          \
    EXPORT void oracle_add_broadcast_fwd_##SFX(const T* x, const T* b, T* y, int rows, int cols) {             \
        add_broadcast_fwd<T>(x, b, y, rows, cols);                                                             \
    }                                                                                                          \
    EXPORT void oracle_add_broadcast_bwd_bias_##SFX(const T* dy, T* db, int rows, int cols) {                  \
        add_broadcast_bwd_bias<T>(dy, db, rows, cols);                                                         \
    }                                                                                                          \
    EXPORT void oracle_softmax_fwd_##SFX(const T* x, T* y, int rows, int cols) { softmax_fwd<T>(x, y, rows, cols); } \
    EXPORT void oracle_softmax_bwd_##SFX(const T* y, const T* dy, T* dx, int rows, int cols) {                 \
        softmax_bwd<T>(y, dy, dx, rows, cols);                                                                 \
    }                                                                                                          \
    EXPORT T oracle_cce_fwd_##SFX(const T* p, const T* t, int rows, int cols) { return cce_fwd<T>(p, t, rows, cols); } \
    EXPORT void oracle_cce_bwd_##SFX(const T* p, const T* t, T* dp, int rows, int cols) { cce_bwd<T>(p, t, dp, rows, cols); } \
    EXPORT T oracle_mse_fwd_##SFX(const T* y, const T* t, int rows, int cols) { return mse_fwd<T>(y, t, rows, cols); } \
    EXPORT void oracle_mse_bwd_##SFX(const T* y, const T* t, T* dy, int rows, int cols) { mse_bwd<T>(y, t, dy, rows, cols); } \
    EXPORT void oracle_matrix_add_##SFX(const T* a, const T* b, T* y, int64_t n) { matrix_add<T>(a, b, y, n); } \
    EXPORT void oracle_matrix_add_three_##SFX(const T* a, const T* b, const T* c, T* y, int64_t n) {           \
        matrix_add_three<T>(a, b, c, y, n);                                                                    \
    }                                                                                                          \
    EXPORT void oracle_matrix_transpose_##SFX(const T* x, T* y, int rows, int cols) { matrix_transpose<T>(x, y, rows, cols); } \
    EXPORT void oracle_layernorm_fwd_##SFX(const T* x, T* y, T* mean, T* stddev, int rows, int cols) {         \
        layernorm_fwd<T>(x, y, mean, stddev, rows, cols);                                                      \
    }                                                                                                          \
    EXPORT void oracle_layernorm_bwd_##SFX(const T* x, const T* mean, const T* stddev, const T* dy, T* dx, int rows, \
                                           int cols) {                                                         \
        layernorm_bwd<T>(x, mean, stddev, dy, dx, rows, cols);                                                 \
    }                                                                                                          \
    EXPORT void oracle_amplified_sigmoid_fwd_##SFX(const T* x, T* y, int64_t n) { amplified_sigmoid_fwd<T>(x, y, n); } \
    EXPORT void oracle_amplified_sigmoid_bwd_##SFX(const T* x, const T* dy, T* dx, int64_t n) {                \
        amplified_sigmoid_bwd<T>(x, dy, dx, n);                                                                \
    }                                                                                                          \
    EXPORT double oracle_time_matmul_fwdbwd_##SFX(int N, int threads, int iters, double* checksum) {           \
        return time_matmul_fwdbwd<T>(N, threads, iters, checksum);                                             \
    }

DEFINE_ENTRY_POINTS(f64, double)
DEFINE_ENTRY_POINTS(f32, float)

EXPORT double oracle_u01(uint64_t seed, uint64_t tensor, uint64_t idx) { return u01(seed, tensor, idx); }
EXPORT int oracle_hardware_threads() { return (int)std::thread::hardware_concurrency(); }
