// MatrixMultiplyAndSumOperation / GpuMatrixMultiplyAndSumOperation
// (src/RMAD/MatrixMultiplyAndSumOperation.cs:50-89, src/RMAD/GpuMatrixMultiplyAndSumOperation.cs:114-154).
//
// Forward: out[0][q] = sum_ij (A . B[q])_ij.  The reference launches its tiled kernel once per
// slice, copies every product back and sums it on the host; here all P products are one
// strided-batched MFMA launch whose epilogue reduces each 128 x 128 tile to one double, so no
// product is ever written to HBM; a second tiny kernel adds the tile sums of each slice.
//
// Backward, as the reference writes it (not the analytic gradient):
//     dB[q] = transpose(A) * dOut[0][q]          (K x M per slice)
//     dA    = sum_q transpose(B[q]) * dOut[0][q]  (q ascending; needs N == M)
// Both are pure data movement: A is read once per group of slices and B exactly once.
#include "common.h"

namespace prad {

template <typename T>
__global__ void __launch_bounds__(64) sum_tiles_kernel(const double* __restrict__ tile_sums, T* __restrict__ out, int64_t tiles,
                                                       int64_t P) {
    const int64_t q = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (q >= P) return;
    double s = 0.0;
    for (int64_t t = 0; t < tiles; ++t) s += tile_sums[q * tiles + t];
    out[q] = (T)s;
}

// S samples (BatchMatrixMultiplyAndSumOperation / BatchGpuMatrixMultiplyAndSumOperation,
// src/RMAD/BatchGpuMatrixMultiplyAndSumOperation.cs:51-74: sample i multiplies its own A[i] with the shared slices B[q]):
// all S x P products are one two-level batch, sample-major like the output (S, 1, P).
template <typename T>
hipError_t launch_matmul_sum_fwd(const T* A, const T* B, T* out, double* workspace, int64_t M, int64_t K, int64_t N, int64_t P,
                                 int64_t S, hipStream_t s) {
    if (P <= 0 || S <= 0) return hipSuccess;
    if (S * P > 65535) return hipErrorInvalidValue;
    GemmArgs<T> g{};
    g.transA = 0; g.transB = 0;
    g.M = M; g.N = N; g.K = K;
    g.A = A; g.lda = K;
    g.B = B; g.ldb = N;
    g.C = nullptr; g.ldc = N;
    g.batch = (int)(S * P);
    g.strideA = 0; g.strideB = K * N; g.strideC = 0;
    if (S > 1) {
        g.batch_inner = (int)P;            // product (sample, slice) = batch index sample * P + slice
        g.strideA = M * K; g.istrideA = 0;
        g.strideB = 0; g.istrideB = K * N;
    }
    g.tile_sums = workspace;
    hipError_t e = launch_gemm<T>(g, s);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((sum_tiles_kernel<T>), dim3((unsigned)((S * P + 63) / 64)), dim3(64), 0, s, workspace, out,
                       gemm_tiles_per_product(M, N), S * P);
    return hipGetLastError();
}

constexpr int TS = 64;       // transpose tile edge
constexpr int Q_PER_WG = 2;  // slices written per workgroup of the dB kernel

// dB[q][k][m] = A[m][k] * dOut[q]: the A tile is transposed through LDS once and scaled into
// Q_PER_WG slices; reads walk k, writes walk m, both contiguous.
template <typename T>
__device__ __forceinline__ void sum_bwd_db_block(T (*tile)[TS + 1], const T* __restrict__ A, const T* __restrict__ dOut,
                                                 T* __restrict__ dB, int64_t M, int64_t K, int64_t P, int64_t bx, int64_t by,
                                                 int64_t bz) {
    const int64_t m0 = bx * TS, k0 = by * TS;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int r = ty; r < TS; r += 4) {
        const int64_t m = m0 + r, k = k0 + tx;
        tile[r][tx] = (m < M && k < K) ? A[m * K + k] : (T)0;
    }
    __syncthreads();
    const int64_t q0 = bz * Q_PER_WG;
    for (int64_t q = q0; q < q0 + Q_PER_WG && q < P; ++q) {
        const T sc = dOut[q];
        T* __restrict__ out = dB + q * K * M;
        for (int r = ty; r < TS; r += 4) {
            const int64_t k = k0 + r, m = m0 + tx;
            if (k < K && m < M) out[k * M + m] = tile[tx][r] * sc;
        }
    }
}

// dA[i][j] = sum_q B[q][j][i] * dOut[q], q ascending, starting from 0 (the reference's
// dA = dA + t).  A thread owns dA elements in the orientation B is stored in (i contiguous), keeps
// their running sums in registers over all q, and the finished tile is transposed through LDS so
// that the single write of dA walks j.
constexpr int TJ = 16;  // rows of B (j) per workgroup of the dA part; 64 columns (i)
template <typename T>
__device__ __forceinline__ void sum_bwd_da_block(T (*tile)[TS + 1], const T* __restrict__ B, const T* __restrict__ dOut,
                                                 T* __restrict__ dA, int64_t M, int64_t K, int64_t N, int64_t P, int64_t bx,
                                                 int64_t by) {
    const int64_t i0 = bx * TS, j0 = by * TJ;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // ty in 0..3, rows ty, ty+4, ty+8, ty+12
    T acc[4] = {(T)0, (T)0, (T)0, (T)0};
    const int64_t i = i0 + tx;
    // Loads of four slices are issued before their (ordered) additions, to keep 16 reads in flight per lane.
    int64_t q = 0;
    for (; q + 4 <= P; q += 4) {
        T b[4][4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const T* __restrict__ Bq = B + (q + u) * K * N;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t j = j0 + ty + 4 * r;
                b[u][r] = (i < N && j < K) ? Bq[j * N + i] : (T)0;
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const T sc = dOut[q + u];
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] = acc[r] + (b[u][r] * sc);
        }
    }
    for (; q < P; ++q) {
        const T sc = dOut[q];
        const T* __restrict__ Bq = B + q * K * N;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int64_t j = j0 + ty + 4 * r;
            const T b = (i < N && j < K) ? Bq[j * N + i] : (T)0;
            acc[r] = acc[r] + (b * sc);
        }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) tile[ty + 4 * r][tx] = acc[r];
    __syncthreads();
    // write dA[i][j]: 16 consecutive j per row i
    const int jj = threadIdx.x & 15, ib = threadIdx.x >> 4;  // ib in 0..15
    for (int r = 0; r < TS; r += 16) {
        const int64_t ii = i0 + ib + r, j = j0 + jj;
        if (ii < M && j < K) dA[ii * K + j] = tile[jj][ib + r];
    }
}

// The same two blocks on 16-byte loads and stores, for operands whose rows are whole, aligned vectors.
template <typename T> struct SumVec;
template <> struct SumVec<double> { typedef double type __attribute__((ext_vector_type(2))); static constexpr int N = 2; };
template <> struct SumVec<float> { typedef float type __attribute__((ext_vector_type(4))); static constexpr int N = 4; };
constexpr int SUM_DA_DEPTH = 32;  // slices of the dA walk in flight per lane (32 x 16 bytes of registers)
constexpr int Q_PER_WG_VEC = 4;  // the transposed tile stays in registers while it is scaled into this many slices

template <typename T>
__device__ __forceinline__ void sum_bwd_db_block_vec(T (*tile)[TS + 1], const T* __restrict__ A, const T* __restrict__ dOut,
                                                     T* __restrict__ dB, int64_t M, int64_t K, int64_t P, int64_t bx, int64_t by,
                                                     int64_t bz) {
    typedef typename SumVec<T>::type V;
    constexpr int VEC = SumVec<T>::N, VPR = TS / VEC, ROWS = 256 / VPR, PASSES = TS / ROWS;
    const int64_t m0 = bx * TS, k0 = by * TS;
    const int t = threadIdx.x, row = t / VPR, col = (t % VPR) * VEC;
    V v[PASSES];
#pragma unroll
    for (int e = 0; e < PASSES; ++e) {
        const int64_t m = m0 + row + e * ROWS, k = k0 + col;
        if (m < M && k < K) v[e] = *reinterpret_cast<const V*>(A + m * K + k);
        else v[e] = (V)(T)0;
    }
#pragma unroll
    for (int e = 0; e < PASSES; ++e)
#pragma unroll
        for (int j = 0; j < VEC; ++j) tile[row + e * ROWS][col + j] = v[e][j];
    __syncthreads();
#pragma unroll
    for (int e = 0; e < PASSES; ++e)
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[e][j] = tile[col + j][row + e * ROWS];  // rows of the output walk k, vectors walk m
    const int64_t q0 = bz * Q_PER_WG_VEC;
    for (int64_t q = q0; q < q0 + Q_PER_WG_VEC && q < P; ++q) {
        const T sc = dOut[q];
        T* __restrict__ out = dB + q * K * M;
#pragma unroll
        for (int e = 0; e < PASSES; ++e) {
            const int64_t k = k0 + row + e * ROWS, m = m0 + col;
            if (k < K && m < M) __builtin_nontemporal_store(v[e] * sc, reinterpret_cast<V*>(out + k * M + m));
        }
    }
}

// DEPTH slices of one (i, j) vector are loaded before their additions, which stay in ascending slice order.
template <typename T, int DEPTH>
__device__ __forceinline__ void sum_da_slices(typename SumVec<T>::type& acc, const T* __restrict__ src, int64_t slice,
                                              const T* __restrict__ dOut, int64_t q, bool inside) {
    typedef typename SumVec<T>::type V;
    V b[DEPTH];
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
        if (inside) b[u] = __builtin_nontemporal_load(reinterpret_cast<const V*>(src + (q + u) * slice));
        else b[u] = (V)(T)0;
    }
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) acc = acc + (b[u] * dOut[q + u]);
}

// 16 vectors (i) x 16 rows (j) of dA^T per workgroup.  The walk over the slices is a chain of load latencies,
// so up to SUM_DA_DEPTH slices are in flight at a time (all of them at the usual slice counts), and what is
// left over goes in halving groups rather than one by one.
template <typename T>
__device__ __forceinline__ void sum_bwd_da_block_vec(T (*tile)[TS + 1], const T* __restrict__ B, const T* __restrict__ dOut,
                                                     T* __restrict__ dA, int64_t M, int64_t K, int64_t N, int64_t P, int64_t bx,
                                                     int64_t by) {
    typedef typename SumVec<T>::type V;
    constexpr int VEC = SumVec<T>::N, IW = 16 * VEC;
    const int64_t i0 = bx * IW, j0 = by * TJ;
    const int t = threadIdx.x, jr = t >> 4, iv = (t & 15) * VEC;
    const int64_t i = i0 + iv, j = j0 + jr;
    const bool inside = i < N && j < K;
    const T* __restrict__ src = B + j * N + i;
    const int64_t slice = K * N;
    V acc = (V)(T)0;
    int64_t q = 0;
    for (; q + SUM_DA_DEPTH <= P; q += SUM_DA_DEPTH) sum_da_slices<T, SUM_DA_DEPTH>(acc, src, slice, dOut, q, inside);
    if (SUM_DA_DEPTH > 16 && q + 16 <= P) { sum_da_slices<T, 16>(acc, src, slice, dOut, q, inside); q += 16; }
    if (SUM_DA_DEPTH > 8 && q + 8 <= P) { sum_da_slices<T, 8>(acc, src, slice, dOut, q, inside); q += 8; }
    if (q + 4 <= P) { sum_da_slices<T, 4>(acc, src, slice, dOut, q, inside); q += 4; }
    if (q + 2 <= P) { sum_da_slices<T, 2>(acc, src, slice, dOut, q, inside); q += 2; }
    if (q < P) sum_da_slices<T, 1>(acc, src, slice, dOut, q, inside);
#pragma unroll
    for (int e = 0; e < VEC; ++e) tile[jr][iv + e] = acc[e];
    __syncthreads();
    const int jj = t & 15, ib = t >> 4;
    for (int r = 0; r < IW; r += 16) {
        const int64_t ii = i0 + ib + r, jo = j0 + jj;
        if (ii < M && jo < K) dA[ii * K + jo] = tile[jj][ib + r];
    }
}

// Both gradients in one launch: the workgroups of the dA part (each walks all P slices) come first in the
// grid, those of the dB part fill in behind them.
template <typename T, bool VECTOR>
__global__ void __launch_bounds__(256) sum_bwd_kernel(const T* __restrict__ A, const T* __restrict__ B, const T* __restrict__ dOut,
                                                      T* __restrict__ dA, T* __restrict__ dB, int64_t M, int64_t K, int64_t N,
                                                      int64_t P, int64_t da_blocks, int64_t da_bm, int64_t bm, int64_t db_by) {
    __shared__ T tile[TS][TS + 1];
    // blockIdx.y is the sample of a batch (its own A, dOut, dA and dB slices; B is shared by all samples)
    const int64_t sample = blockIdx.y;
    A += sample * M * K;
    dOut += sample * P;
    if (dA != nullptr) dA += sample * M * K;
    if (dB != nullptr) dB += sample * P * K * M;
    int64_t id = blockIdx.x;
    if (id < da_blocks) {
        if (VECTOR) sum_bwd_da_block_vec<T>(tile, B, dOut, dA, M, K, N, P, id % da_bm, id / da_bm);
        else sum_bwd_da_block<T>(tile, B, dOut, dA, M, K, N, P, id % da_bm, id / da_bm);
        return;
    }
    id -= da_blocks;
    if (VECTOR) sum_bwd_db_block_vec<T>(tile, A, dOut, dB, M, K, P, id % bm, (id / bm) % db_by, id / (bm * db_by));
    else sum_bwd_db_block<T>(tile, A, dOut, dB, M, K, P, id % bm, (id / bm) % db_by, id / (bm * db_by));
}

template <typename T>
hipError_t launch_matmul_sum_bwd(const T* A, const T* B, const T* dOut, T* dA, T* dB, int64_t M, int64_t K, int64_t N, int64_t P,
                                 int64_t S, hipStream_t s) {
    if (M <= 0 || K <= 0 || S <= 0) return hipSuccess;
    if (S > 65535) return hipErrorInvalidValue;
    constexpr int VEC = SumVec<T>::N;
    auto aligned = [](const void* p) { return p == nullptr || reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    const bool vec = M % VEC == 0 && K % VEC == 0 && N % VEC == 0 && aligned(A) && aligned(B) && aligned(dA) && aligned(dB);
    const int64_t iw = vec ? 16 * VEC : TS, qpw = vec ? Q_PER_WG_VEC : Q_PER_WG;
    const int64_t bm = (M + TS - 1) / TS, db_by = (K + TS - 1) / TS, da_bm = (M + iw - 1) / iw;
    const int64_t da_blocks = dA != nullptr ? da_bm * ((K + TJ - 1) / TJ) : 0;
    const int64_t db_blocks = (dB != nullptr && P > 0) ? bm * db_by * ((P + qpw - 1) / qpw) : 0;
    if (da_blocks + db_blocks == 0) return hipSuccess;
    if (da_blocks + db_blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)(da_blocks + db_blocks), (unsigned)S), block(256);
    if (vec)
        hipLaunchKernelGGL((sum_bwd_kernel<T, true>), grid, block, 0, s, A, B, dOut, dA, dB, M, K, N, P, da_blocks, da_bm, bm, db_by);
    else
        hipLaunchKernelGGL((sum_bwd_kernel<T, false>), grid, block, 0, s, A, B, dOut, dA, dB, M, K, N, P, da_blocks, da_bm, bm, db_by);
    return hipGetLastError();
}

template hipError_t launch_matmul_sum_fwd<double>(const double*, const double*, double*, double*, int64_t, int64_t, int64_t,
                                                  int64_t, int64_t, hipStream_t);
template hipError_t launch_matmul_sum_fwd<float>(const float*, const float*, float*, double*, int64_t, int64_t, int64_t, int64_t,
                                                 int64_t, hipStream_t);
template hipError_t launch_matmul_sum_bwd<double>(const double*, const double*, const double*, double*, double*, int64_t, int64_t,
                                                  int64_t, int64_t, int64_t, hipStream_t);
template hipError_t launch_matmul_sum_bwd<float>(const float*, const float*, const float*, float*, float*, int64_t, int64_t,
                                                 int64_t, int64_t, int64_t, hipStream_t);

}  // namespace prad
