/*
 * prad_hip.h -- C ABI of libprad_hip.so: gfx950 (MI355X) implementation of
 * ParallelReverseAutoDiff's matrix-multiply forward/backward path and the gradient kernels
 * around it (activation backward, gradient clip, Adam).
 *
 * Conventions
 *   - Every function returns an int32 status (PRAD_OK == 0, negative on failure) unless it is
 *     documented as a plain getter.  No exception or abort crosses this boundary;
 *     prad_last_error() returns the calling thread's last failure message.
 *   - Matrices are dense row-major device buffers behind opaque handles (prad_buf_t).  A handle
 *     is valid on any host thread.  The reference's jagged Matrix (one array per row) is
 *     marshalled once with prad_buf_upload_rows and stays resident.
 *   - All work is enqueued, in call order, on one library stream under one lock; calls may come from
 *     any number of host threads (the reference runs Backward of different operations concurrently
 *     on pool threads, src/RMAD/OperationNeuralNetworkVisitor.cs:303-306) and execute in the order in
 *     which they took the lock.  Downloads and prad_stream_sync wait for the stream.  While one
 *     thread records a launch sequence (prad_graph_begin .. prad_graph_end), calls from other threads
 *     return PRAD_ERR_RECORDING and enqueue nothing.
 *   - Kernels that need device scratch (products split along K, clip statistics, loss partial sums,
 *     tall column sums) share one workspace that grows on demand.  A recorded launch sequence keeps
 *     the workspace address it was recorded with: an outgrown workspace is kept alive until the last
 *     recorded sequence is destroyed, and growing it during a recording fails (run the sequence once
 *     eagerly first).
 *   - dtype: PRAD_F64 restates the PRAD (double) build, PRAD_F32 the PRADLite (float) build.
 *
 * Citations are to the reference tree (ameritusweb/ParallelReverseAutoDiff).
 */
#ifndef PRAD_HIP_H
#define PRAD_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    PRAD_OK = 0,
    PRAD_ERR_NOT_INITIALIZED = -1, /* CudaNotInitializedException, src/RMAD/GpuMatrixMultiplyOperation.cs:115-118 */
    PRAD_ERR_SHAPE = -2,           /* InvalidOperationException("Input 1 columns do not match Input 2 rows"), src/RMAD/MatrixMultiplyOperation.cs:59-62 */
    PRAD_ERR_ALLOC = -3,
    PRAD_ERR_LAUNCH = -4,          /* InvalidOperationException("CUBLAS failure."), src/RMAD/CudaBlas.cs:251-256 */
    PRAD_ERR_BAD_HANDLE = -5,
    PRAD_ERR_ARG = -6,             /* ArgumentException, src/RMAD/GpuMatrixMultiplyOperation.cs:177-180 */
    PRAD_ERR_NOT_RECTANGULAR = -7, /* InvalidOperationException("The given jagged array is not rectangular."), src/RMAD/GpuMatrixMultiplyOperation.cs:244-247 */
    PRAD_ERR_DTYPE = -8,
    PRAD_ERR_RECORDING = -9        /* refused because of an open recording (prad_graph_begin): the call came from another
                                      thread, or it allocates, copies to or from the host or waits for the device */
};

enum { PRAD_F64 = 0, PRAD_F32 = 1 };

/* Activation selector for the elementwise backward kernels and the fused GEMM epilogues.
 * `src` is what the reference operation caches: its input x or its output y. */
enum {
    PRAD_ACT_NONE = 0,
    PRAD_ACT_LEAKYRELU = 1, /* src = x; src/RMAD/LeakyReLUOperation.cs:54-93 */
    PRAD_ACT_SIGMOID = 2,   /* src = y; src/RMAD/SigmoidOperation.cs:46-84 */
    PRAD_ACT_TANH = 3,      /* src = y; src/RMAD/TanhOperation.cs:42-79 */
    PRAD_ACT_GELU = 4,      /* src = x; src/RMAD/GELUOperation.cs:44-101 (the reference's own derivative formula) */
    PRAD_ACT_AMPLIFIED_SIGMOID = 5 /* src = x; src/RMAD/AmplifiedSigmoidOperation.cs:44-84 (derivative as written there) */
};

typedef struct prad_buf* prad_buf_t;

/* ---- lifecycle: replaces CudaBlas.Instance.{DeviceId,Initialize,Dispose,IsInitialized},
 *      src/RMAD/CudaBlas.cs:71-155 ------------------------------------------------------- */
int32_t prad_init(int32_t device_id);
int32_t prad_shutdown(void);
int32_t prad_is_initialized(void); /* getter: 1 or 0 */
int32_t prad_device_id(void);      /* getter: device passed to prad_init, -1 before */
const char* prad_last_error(void); /* getter: thread-local, never NULL */
int32_t prad_stream_sync(void);
void* prad_stream(void);           /* getter: the library's hipStream_t, for callers that record their own events */

/* ---- device-resident matrices: replace the per-call To2D / Allocate2DDenseX / CopyFromCPU /
 *      GetAsArray2D / ToJagged of src/RMAD/GpuMatrixMultiplyOperation.cs:170-271 ----------- */
int32_t prad_buf_alloc(int32_t dtype, int64_t rows, int64_t cols, prad_buf_t* out); /* zero-filled, like new Matrix(rows, cols) */
int32_t prad_buf_alloc_deep(int32_t dtype, int64_t depth, int64_t rows, int64_t cols, prad_buf_t* out); /* DeepMatrix: depth contiguous slices; src/RMAD/DeepMatrix.cs:22 */
/* The same without the zero fill, for an output that the next call overwrites whole (a product with accumulate == 0, an
 * activation, a transpose): the fresh output Matrix every Forward / Backward of the reference allocates
 * (e.g. src/RMAD/MatrixMultiplyOperation.cs:64, :91, :107) without a launch spent on zeros that are never read.
 * Contents are undefined until written. */
int32_t prad_buf_alloc_output(int32_t dtype, int64_t depth, int64_t rows, int64_t cols, prad_buf_t* out);
int32_t prad_buf_wrap(int32_t dtype, int64_t rows, int64_t cols, void* device_ptr, prad_buf_t* out); /* borrow caller-owned device memory */
int32_t prad_buf_wrap_deep(int32_t dtype, int64_t depth, int64_t rows, int64_t cols, void* device_ptr, prad_buf_t* out); /* the same for depth contiguous slices (a tensor of more than two dimensions: Tensor.Shape, src/PRAD/Tensor.cs) */
/* Owned device memory goes back to a pool inside the library, by size class, without waiting for the device and
 * without hipFree: the reference's pattern is a fresh output Matrix per operation per step, released by the garbage
 * collector (src/RMAD/GpuMatrixMultiplyOperation.cs:190-201 allocates and drops three device arrays per call), and the
 * next allocation of the class takes the block back.  One in-order stream makes the reuse safe.  A buffer that a
 * recorded launch sequence addresses must outlive the sequence. */
int32_t prad_buf_free(prad_buf_t b);
/* Gives the pooled blocks back to the device (waits for the stream).  The pool also releases them by itself when an
 * allocation would otherwise fail, and never holds more than half of the device memory (PRAD_POOL_MAX_BYTES overrides). */
int32_t prad_pool_trim(void);
/* Counters since the library was loaded, any of which may be NULL: hipMalloc calls and hipFree calls for matrices,
 * waits for the stream, allocations served from the pool, bytes the pool holds now.  For tests and tuning: a training
 * step in its steady state adds nothing to the first three. */
int32_t prad_alloc_stats(int64_t* device_mallocs, int64_t* device_frees, int64_t* stream_syncs, int64_t* pool_hits,
                         int64_t* pooled_bytes);
int32_t prad_buf_shape(prad_buf_t b, int64_t* depth, int64_t* rows, int64_t* cols, int32_t* dtype);
void* prad_buf_device_ptr(prad_buf_t b); /* getter: NULL for a bad handle */
int32_t prad_buf_zero(prad_buf_t b);
/* GradientClearer.Clear over a model's layers (src/RMAD/GradientClearer.cs:21-86): n buffers zeroed by one launch (one per
 * 40 buffers). */
int32_t prad_zero_multi(const prad_buf_t* bufs, int32_t n);
/* Jagged upload: row_ptrs[i] points at row i (cols elements).  row_lengths may be NULL; when given,
 * any length != cols fails with PRAD_ERR_NOT_RECTANGULAR. For a deep buffer pass depth*rows pointers. */
int32_t prad_buf_upload_rows(prad_buf_t b, const void* const* row_ptrs, const int64_t* row_lengths);
int32_t prad_buf_download_rows(prad_buf_t b, void* const* row_ptrs);
int32_t prad_buf_upload(prad_buf_t b, const void* src, int64_t ld);  /* contiguous rows, ld elements apart */
int32_t prad_buf_download(prad_buf_t b, void* dst, int64_t ld);
int32_t prad_buf_copy(prad_buf_t dst, prad_buf_t src);

/* ---- matrix multiply: MatrixMultiplyOperation.Forward / Backward,
 *      src/RMAD/MatrixMultiplyOperation.cs:50-80 and :83-126 (same contract as
 *      GpuMatrixMultiplyOperation.cs:113-161 and CudaMatrixMultiplyOperation.cs:51-96) ------ */
/* C[M x N] = A[M x K] . B[K x N] */
int32_t prad_matmul_fwd(prad_buf_t A, prad_buf_t B, prad_buf_t C);
/* dA[M x K] = dC . B^T ; dB[K x N] = A^T . dC.  dA or dB may be NULL to skip that product.
 * accumulate_dA / accumulate_dB != 0 adds into the destination instead of overwriting it
 * (the dest += grad of OperationBase.AccumulateGradient, src/RMAD/OperationBase.cs:295-303).
 * When both are requested for a small layer they may share one launch; the results are those of
 * the two products computed one after the other, bit for bit (a dA that overlaps dC, A or dB in
 * memory is always computed first, in a launch of its own). */
int32_t prad_matmul_bwd(prad_buf_t dC, prad_buf_t A, prad_buf_t B, prad_buf_t dA, prad_buf_t dB,
                        int32_t accumulate_dA, int32_t accumulate_dB);
/* Forward with the next operations of the graph fused into the product's epilogue:
 * Z = A.B + bias (bias 1 x N, may be NULL: MatrixAddBroadcastingOperation.cs:32-54), H = act(Z).
 * Z (may be NULL) receives the pre-activation the activation's Backward caches, H the output. */
int32_t prad_matmul_fwd_fused(prad_buf_t A, prad_buf_t B, prad_buf_t bias, prad_buf_t Z, prad_buf_t H,
                              int32_t act, double alpha);
/* Backward with the upstream activation's Backward fused into the dA product:
 * dA = (dC . B^T) (.) act'(act_src), act_src shaped like dA. */
int32_t prad_matmul_bwd_fused(prad_buf_t dC, prad_buf_t A, prad_buf_t B, prad_buf_t dA, prad_buf_t dB,
                              int32_t accumulate_dB, int32_t act, prad_buf_t act_src, double alpha);
/* Backward of the pair MatrixMultiply -> MatrixAddBroadcasting (a layer's Z = A.B + bias) for the
 * upstream gradient dC of Z: dB = A^T . dC, dbias = column sums of dC
 * (src/RMAD/MatrixAddBroadcastingOperation.cs:57-70), dA = (dC . B^T) (.) act'(act_src) with
 * act = PRAD_ACT_NONE for a plain dA.  dA, dB, dbias may each be NULL.  The column sum shares the
 * launch of the dB product (both read dC only), so the pair costs two launches. */
int32_t prad_matmul_bias_bwd(prad_buf_t dC, prad_buf_t A, prad_buf_t B, prad_buf_t dA, prad_buf_t dB, prad_buf_t dbias,
                             int32_t accumulate_dB, int32_t act, prad_buf_t act_src, double alpha);
/* General product on handles: C = op(A).op(B) (+ C when accumulate).  trans flags are 0/1.
 * Supported: (0,0), (0,1), (1,0). */
int32_t prad_gemm(int32_t transA, int32_t transB, prad_buf_t A, prad_buf_t B, prad_buf_t C, int32_t accumulate);
/* Strided batched product over the slices of deep buffers (BatchMatrixMultiplyOperation and
 * BatchGpuMatrixMultiplyOperation, src/RMAD/BatchGpuMatrixMultiplyOperation.cs:56-143).  A buffer of
 * depth 1 is broadcast to every slice. */
int32_t prad_gemm_batched(int32_t transA, int32_t transB, prad_buf_t A, prad_buf_t B, prad_buf_t C, int32_t accumulate);

/* Raw device-pointer entry points (row-major, leading dimensions in elements, library stream). */
int32_t prad_gemm_f64(int32_t transA, int32_t transB, int64_t M, int64_t N, int64_t K, const double* A, int64_t lda,
                      const double* B, int64_t ldb, double* C, int64_t ldc, int32_t accumulate);
int32_t prad_gemm_f32(int32_t transA, int32_t transB, int64_t M, int64_t N, int64_t K, const float* A, int64_t lda,
                      const float* B, int64_t ldb, float* C, int64_t ldc, int32_t accumulate);

/* Strided batched product on raw device pointers: `batch` products, operand b at base + b * stride (elements;
 * stride 0 shares an operand).  This is the form the per-window, per-head products of an attention block
 * take, and the one a batched Tensor.MatrixMultiply (src/PRAD/Tensor.cs:572-608, which rejects more than
 * two dimensions today) would bind. */
int32_t prad_gemm_strided_batched_f64(int32_t transA, int32_t transB, int64_t M, int64_t N, int64_t K, const double* A,
                                      int64_t lda, int64_t strideA, const double* B, int64_t ldb, int64_t strideB, double* C,
                                      int64_t ldc, int64_t strideC, int32_t batch, int32_t accumulate);
int32_t prad_gemm_strided_batched_f32(int32_t transA, int32_t transB, int64_t M, int64_t N, int64_t K, const float* A,
                                      int64_t lda, int64_t strideA, const float* B, int64_t ldb, int64_t strideB, float* C,
                                      int64_t ldc, int64_t strideC, int32_t batch, int32_t accumulate);
/* Two-level batches (attention: windows x heads) in one launch: product (o, i), o < batch_outer, i < batch_inner,
 * takes its operand blocks at o * stride + i * istride elements from the base pointers. */
int32_t prad_gemm_strided_batched_2d_f64(int32_t transA, int32_t transB, int64_t M, int64_t N, int64_t K, const double* A,
                                         int64_t lda, int64_t strideA, int64_t istrideA, const double* B, int64_t ldb,
                                         int64_t strideB, int64_t istrideB, double* C, int64_t ldc, int64_t strideC,
                                         int64_t istrideC, int32_t batch_outer, int32_t batch_inner, int32_t accumulate);
int32_t prad_gemm_strided_batched_2d_f32(int32_t transA, int32_t transB, int64_t M, int64_t N, int64_t K, const float* A,
                                         int64_t lda, int64_t strideA, int64_t istrideA, const float* B, int64_t ldb,
                                         int64_t strideB, int64_t istrideB, float* C, int64_t ldc, int64_t strideC,
                                         int64_t istrideC, int32_t batch_outer, int32_t batch_inner, int32_t accumulate);

/* One-shot host-pointer forms with today's call-per-operation behaviour of
 * GpuMatrixMultiplyOperation.Forward/Backward (src/RMAD/GpuMatrixMultiplyOperation.cs:113-161):
 * jagged rows in, jagged rows out, synchronous. */
int32_t prad_matmul_fwd_host(int32_t dtype, const void* const* a_rows, const void* const* b_rows, void* const* c_rows,
                             int64_t M, int64_t K, int64_t K2, int64_t N);
int32_t prad_matmul_bwd_host(int32_t dtype, const void* const* dc_rows, const void* const* a_rows,
                             const void* const* b_rows, void* const* da_rows, void* const* db_rows, int64_t M,
                             int64_t K, int64_t N);

/* ---- the tape engine's products on flat row-major arrays (no jagged marshalling):
 *      Tensor.MatrixMultiply, src/PRAD/Tensor.cs:572-608: c (m x n) = alpha * a (m x k) . b (k2 x n); the reference's
 *      beta multiplies a freshly zeroed result and has no effect, so it is not a parameter; k != k2 is the
 *      reference's ArgumentException("Incompatible shapes for matrix multiplication.") (status PRAD_ERR_SHAPE).
 *      TensorReverse.MatrixMultiplyReverse, src/PRAD/TensorReverse.cs:94-157: da = dc . b^T, db = a^T . dc.
 *      Device-resident tensors use prad_buf_upload / prad_matmul_fwd / prad_matmul_bwd or prad_gemm_f64/f32
 *      on their own device pointers. */
int32_t prad_tensor_matmul_host(int32_t dtype, const void* a, const void* b, void* c, int64_t m, int64_t k, int64_t k2,
                                int64_t n, double alpha);
int32_t prad_tensor_matmul_reverse_host(int32_t dtype, const void* dc, const void* a, const void* b, void* da, void* db,
                                        int64_t m, int64_t k, int64_t n);

/* ---- MatrixMultiplyAndSumOperation / GpuMatrixMultiplyAndSumOperation,
 *      src/RMAD/MatrixMultiplyAndSumOperation.cs:50-89, GpuMatrixMultiplyAndSumOperation.cs:114-154, and their per-sample
 *      wrappers BatchMatrixMultiplyAndSumOperation / BatchGpuMatrixMultiplyAndSumOperation
 *      (src/RMAD/BatchGpuMatrixMultiplyAndSumOperation.cs:51-74): A of depth S holds one M x K matrix per sample, the P
 *      slices of B (K x N) are shared by all samples; S = 1 is the single operation. */
/* out[i][0][q] = sum over all entries of A[i] . B[q]; out is deep (S, 1, P).  One launch over all S * P products. */
int32_t prad_matmul_sum_fwd(prad_buf_t A, prad_buf_t B, prad_buf_t out);
/* As written in the reference, per sample i: dB[i * P + q] = A[i]^T * dOut[i][0][q] (dB deep (S * P, K, M));
 * dA[i] = sum_q B[q]^T * dOut[i][0][q] (dA deep (S, M, K); needs N == M).  dA or dB may be NULL.  One launch. */
int32_t prad_matmul_sum_bwd(prad_buf_t A, prad_buf_t B, prad_buf_t dOut, prad_buf_t dA, prad_buf_t dB);
/* Independent products summed into one output plus a broadcast bias: C = sum_q A[q].B[q] + bias, A deep
 * (P, M, K), B deep (P, K, N), bias 1 x N or NULL, C M x N.  The reference has no single operation of this
 * form (it composes MatrixMultiplyOperation.Forward, src/RMAD/MatrixMultiplyOperation.cs:50-80, a sum of
 * matrices and MatrixAddBroadcastingOperation.cs:32-54); results are those of that composition with the
 * products added in slice order.  Backward for the upstream gradient dC: dA[q] = dC . B[q]^T,
 * dB[q] = A[q]^T . dC, dbias = column sums of dC; each may be NULL. */
int32_t prad_matmul_batch_sum_fwd(prad_buf_t A, prad_buf_t B, prad_buf_t bias, prad_buf_t C);
int32_t prad_matmul_batch_sum_bwd(prad_buf_t dC, prad_buf_t A, prad_buf_t B, prad_buf_t dA, prad_buf_t dB, prad_buf_t dbias);

/* ---- elementwise forward / backward (bandwidth kernels) ------------------------------------- */
int32_t prad_act_fwd(int32_t act, prad_buf_t x, prad_buf_t y, double alpha);
/* dx = dy (.) act'(src); src is x for LeakyReLU/GELU/AmplifiedSigmoid and y for Sigmoid/Tanh. */
int32_t prad_act_bwd(int32_t act, prad_buf_t src, prad_buf_t dy, prad_buf_t dx, double alpha);
/* HadamardProductOperation, src/RMAD/HadamardProductOperation.cs:50-118 */
int32_t prad_hadamard_fwd(prad_buf_t a, prad_buf_t b, prad_buf_t y);
int32_t prad_hadamard_bwd(prad_buf_t a, prad_buf_t b, prad_buf_t dy, prad_buf_t da, prad_buf_t db);
/* y = x * scalar, MatrixMultiplyScalarOperation.Forward and (with dy for x) Backward, src/RMAD/MatrixMultiplyScalarOperation.cs */
int32_t prad_scale(prad_buf_t x, prad_buf_t y, double scalar);
/* dest += grad, src/RMAD/OperationBase.cs:295-303 */
int32_t prad_accumulate(prad_buf_t dest, prad_buf_t grad);
/* y = x + bias broadcast over rows; db[0][j] = sum_i dy[i][j]; src/RMAD/MatrixAddBroadcastingOperation.cs:32-70 */
int32_t prad_add_broadcast_fwd(prad_buf_t x, prad_buf_t bias, prad_buf_t y);
int32_t prad_add_broadcast_bwd_bias(prad_buf_t dy, prad_buf_t dbias);
/* MatrixAddOperation.Forward, src/RMAD/MatrixAddOperation.cs:30-45 (Backward returns dy for both inputs), and
 * MatrixAddThreeOperation.Forward, src/RMAD/MatrixAddThreeOperation.cs:35-50: y = (a + b) + c. */
int32_t prad_add(prad_buf_t a, prad_buf_t b, prad_buf_t y);
int32_t prad_add_three(prad_buf_t a, prad_buf_t b, prad_buf_t c, prad_buf_t y);
/* MatrixTransposeOperation, src/RMAD/MatrixTransposeOperation.cs:30-64: y (cols x rows) = x^T; Backward is the
 * same call on dy. */
int32_t prad_transpose(prad_buf_t x, prad_buf_t y);
/* LayerNormalizationOperation, src/RMAD/LayerNormalizationOperation.cs:56-110: per row, y = (x - mean) /
 * (stddev + 1e-9) with the population deviation; mean and stddev (1 x rows) are what the operation caches.
 * Backward as written there: dx = dy * ((1 - 1/cols) / (stddev + eps) - (x - mean)^2 / (cols * (stddev + eps)^3)). */
int32_t prad_layernorm_fwd(prad_buf_t x, prad_buf_t y, prad_buf_t mean, prad_buf_t stddev);
int32_t prad_layernorm_bwd(prad_buf_t x, prad_buf_t mean, prad_buf_t stddev, prad_buf_t dy, prad_buf_t dx);

/* ---- operations that close a training step on the device ------------------------------------ */
/* Row-wise softmax, src/RMAD/SoftmaxOperation.cs:45-110 (backward: dx = J^T . dy per row). */
int32_t prad_softmax_fwd(prad_buf_t x, prad_buf_t y);
int32_t prad_softmax_bwd(prad_buf_t y, prad_buf_t dy, prad_buf_t dx);
/* MatrixMultiplyScalarOperation followed by SoftmaxOperation in one pass, as attention scores take them
 * (src/RMAD/MatrixMultiplyScalarOperation.cs, src/RMAD/SoftmaxOperation.cs:45-110): y = softmax(alpha * x) and,
 * backward through both, dx = alpha * (J^T . dy).  Same values as prad_scale + prad_softmax_fwd and
 * prad_softmax_bwd + prad_scale. */
int32_t prad_softmax_scaled_fwd(prad_buf_t x, double alpha, prad_buf_t y);
int32_t prad_softmax_scaled_bwd(prad_buf_t y, prad_buf_t dy, double alpha, prad_buf_t dx);
/* Categorical cross-entropy, src/RMAD/Loss/CategoricalCrossEntropyLossOperation.cs:37-86:
 * loss (1 x 1) = sum(-t * log(p + 1e-15)) / rows ; dp = -(1/rows) * t / (p + 1e-15). */
int32_t prad_cce_fwd(prad_buf_t p, prad_buf_t target, prad_buf_t loss);
int32_t prad_cce_bwd(prad_buf_t p, prad_buf_t target, prad_buf_t dp);

/* Mean squared error, src/RMAD/Loss/MeanSquaredErrorLossOperation.cs:
 * loss (1 x 1) = sum((y - t)^2) / (rows*cols) ; dy = (2 / (rows*cols)) * (y - t). */
int32_t prad_mse_fwd(prad_buf_t y, prad_buf_t target, prad_buf_t loss);
int32_t prad_mse_bwd(prad_buf_t y, prad_buf_t target, prad_buf_t dy);
/* Forward and Backward of MeanSquaredErrorLossOperation in one pass over y and target (the loss of prad_mse_fwd
 * and the gradient of prad_mse_bwd, value for value). */
int32_t prad_mse(prad_buf_t y, prad_buf_t target, prad_buf_t loss, prad_buf_t dy);
/* One LSTM time step's pointwise part, fused.  The reference builds it from separate nodes: three
 * SigmoidOperation and two TanhOperation forward (src/RMAD/SigmoidOperation.cs:46-62, TanhOperation.cs:42-57),
 * three HadamardProductOperation (HadamardProductOperation.cs:50-81) and a MatrixAddOperation (MatrixAddOperation.cs:29-45).
 * G (rows x 4*hidden, gate blocks [i|f|g|o]) holds the pre-activations and is overwritten with the activated
 * gates; c = f.c_prev + i.g ; tanh_c = tanh(c) ; h = o.tanh_c. */
int32_t prad_lstm_cell_fwd(prad_buf_t G, prad_buf_t c_prev, prad_buf_t c, prad_buf_t tanh_c, prad_buf_t h);
/* Backward of the same nodes (their Backward methods, same files): dh = dh_a + dh_b (dh_b may be NULL),
 * dc_in (may be NULL) is the cell-state gradient arriving from the next step; writes dG (rows x 4*hidden,
 * gradient of the pre-activations) and dc_prev. */
int32_t prad_lstm_cell_bwd(prad_buf_t gates, prad_buf_t c_prev, prad_buf_t tanh_c, prad_buf_t dh_a, prad_buf_t dh_b,
                           prad_buf_t dc_in, prad_buf_t dG, prad_buf_t dc_prev);
/* One time step in one launch each way (the recurrent product with the cell arithmetic as its epilogue; same
 * results as the product followed by prad_lstm_cell_fwd / preceded by prad_lstm_cell_bwd):
 * forward: G (rows x 4*hidden, holding x_t . W_x + b) becomes the activated gates of G + h_prev . Wh, and c, tanh_c, h
 * are written; backward for step t: dh = dh_loss + dG_next . Wh^T (dG_next = gate gradients of step t + 1), then the
 * cell's backward writes dG and dc_prev.  dc_in may be NULL.  dh_scratch (rows x hidden) is only written when the
 * shape needs the two-launch path (hidden not a multiple of the kernels' K slab, unaligned buffers). */
int32_t prad_lstm_step_fwd(prad_buf_t h_prev, prad_buf_t Wh, prad_buf_t G, prad_buf_t c_prev, prad_buf_t c, prad_buf_t tanh_c,
                           prad_buf_t h);
int32_t prad_lstm_step_bwd(prad_buf_t dG_next, prad_buf_t Wh, prad_buf_t gates, prad_buf_t c_prev, prad_buf_t tanh_c,
                           prad_buf_t dh_loss, prad_buf_t dc_in, prad_buf_t dG, prad_buf_t dc_prev, prad_buf_t dh_scratch);
/* All time steps of a sequence in one launch each way.  The reference unrolls a sequence into one set of operation
 * nodes per time step (src/RMAD/ComputationGraph.cs:808-849), each step's recurrent product being a
 * MatrixMultiplyOperation (src/RMAD/MatrixMultiplyOperation.cs:50-126) that needs the step before it; these two run
 * that loop inside one kernel, with the recurrent weight held in registers for the whole sequence and the time
 * steps ordered by flags between the workgroups of a group of 16 batch rows.  Same values as `steps` calls of
 * prad_lstm_step_fwd / prad_lstm_step_bwd up to the order of the sums along hidden (forward) and 4*hidden (backward).
 *   forward:  G (steps*batch x 4*hidden) holds x_t . W_x + b for every step and becomes the activated gates;
 *             C and Hs ((steps+1)*batch x hidden) hold c_0 / h_0 in their first batch rows and receive c_t / h_t in
 *             the following blocks; tanh_c (steps*batch x hidden) receives tanh(c_t).
 *   backward: dh_loss (steps*batch x hidden) is the loss gradient with respect to every h_t; dG receives the gradient of
 *             the pre-activations of every step.  (dh_{-1} and dc_{-1}, which nothing consumes, are not formed.)
 * The one-launch kernels take float, batch a multiple of 16, hidden a multiple of 64 up to 512, and need
 * (batch/16)*(hidden/16) workgroups on the device at once, one per compute unit: prad_lstm_sequence_supported says 1 or 0
 * for a shape (0 for every shape once the kernels are off, see below).  Every other shape and element type, and every
 * call while the kernels are off, runs the same sequence as one launch per time step inside these two calls
 * (prad_lstm_step_fwd / prad_lstm_step_bwd on windows of the same buffers), so the calls are always valid.
 * Whether the device holds the whole grid is asked, not assumed: the first call for a grid larger than any before runs a
 * probe kernel of the same grid and footprint that only takes a roll call, and waits for it (once per process and grid
 * size; inside a recording an unproven grid takes the per-step path).  A probe that fails - another process or a
 * compute-unit mask holds compute units - turns the kernels off, leaves a note in prad_last_error and the call goes on
 * per time step and returns PRAD_OK.  Every wait inside the kernels is bounded as well (PRAD_LSTM_SPIN_LIMIT polls,
 * default 2^22): if compute units are taken away later, the kernels end early, the next call that waits for the stream
 * returns PRAD_ERR_LAUNCH (what was computed since the last successful wait is invalid), and the kernels stay off from
 * then on.  prad_lstm_sequence_enable(1) turns them back on (the next call probes again), (0) turns them off;
 * PRAD_LSTM_SEQUENCE=0 in the environment starts with them off.  A recorded launch sequence keeps the path it was
 * recorded with. */
int32_t prad_lstm_sequence_supported(int32_t dtype, int64_t batch, int64_t hidden, int64_t steps);
int32_t prad_lstm_sequence_enable(int32_t on);
int32_t prad_lstm_sequence_fwd(prad_buf_t Wh, prad_buf_t G, prad_buf_t C, prad_buf_t Hs, prad_buf_t tanh_c, int64_t steps);
int32_t prad_lstm_sequence_bwd(prad_buf_t Wh, prad_buf_t gates, prad_buf_t C, prad_buf_t tanh_c, prad_buf_t dh_loss, prad_buf_t dG,
                               int64_t steps);
/* Windowed self-attention of a block, forward, in one launch: per window w and head h,
 * S = Q_wh . K_wh^T * scale, P = softmax rows(S), O_wh = P . V_wh - the nodes MatrixMultiply, MatrixMultiplyScalar, Softmax,
 * MatrixMultiply of examples/swin/SwinExample/SwinTransformerTools.cs:348-399 (src/RMAD/MatrixMultiplyOperation.cs:50-86,
 * src/RMAD/SoftmaxOperation.cs:45-110).  QKV is (windows*tokens) x (3*heads*head_dim), rows window-major, columns
 * [Q | K | V] with a head's head_dim columns inside each; P (heads*windows*tokens x tokens, head-major: what the backward
 * pass reads) and O ((windows*tokens) x (heads*head_dim)) are written; the scores themselves never reach memory.  Same
 * values as prad_gemm_strided_batched_2d_f32 + prad_softmax_scaled_fwd + prad_gemm_strided_batched_2d_f32 up to the order
 * of the sums along head_dim.  Float, head_dim 32, at most 64 tokens per window: prad_window_attention_supported says
 * 1 or 0, the call returns PRAD_ERR_ARG for other shapes. */
int32_t prad_window_attention_supported(int32_t dtype, int64_t tokens, int64_t head_dim);
int32_t prad_window_attention_fwd(prad_buf_t QKV, prad_buf_t P, prad_buf_t O, int64_t windows, int64_t heads, int64_t tokens, double scale);
/* Backward of the same nodes in one launch: from dO (the gradient of O) and the forward's P,
 * dP = dO . V^T, dV = P^T . dO, dS = P (.) (dP - rowsum(dP (.) P)) * scale (src/RMAD/SoftmaxOperation.cs:75-110 and the
 * scalar product's backward), dQ = dS . K, dK = dS^T . Q (src/RMAD/MatrixMultiplyOperation.cs:88-143); dQKV
 * ((windows*tokens) x (3*heads*head_dim), columns [dQ | dK | dV]) is written whole, dP and dS never reach memory.  Same
 * values as the five separate calls up to the order of the sums.  Shapes as for the forward call. */
int32_t prad_window_attention_bwd(prad_buf_t QKV, prad_buf_t P, prad_buf_t dO, prad_buf_t dQKV, int64_t windows, int64_t heads, int64_t tokens,
                                  double scale);
/* Borrowed view of rows [row0, row0 + rows) of a 2-D buffer (a block of a fused weight, a time step of a
 * stacked sequence).  The view must be freed before its parent. */
int32_t prad_buf_view_rows(prad_buf_t parent, int64_t row0, int64_t rows, prad_buf_t* out);

/* ---- replay of a fixed launch sequence: everything enqueued by the calling thread between begin and end
 *      is recorded instead of executed and can then be launched as one submission.  The forward loop
 *      of the reference walks the same operation list every step
 *      (examples/feedforward/ParallelReverseAutoDiff.FeedForwardExample/FeedForwardNeuralNetwork.cs:212-303);
 *      a recorded step replaces ~20 launches by one.  Entry points that allocate, free, copy to or from the
 *      host or wait for the device return PRAD_ERR_RECORDING while a recording is open, and so does every
 *      enqueueing call from a thread other than the recording one.
 *      AdamIteration: the reference's caller advances it once per step (AdamOptimizer.cs:204-207, set from the
 *      iteration count at FeedForwardNeuralNetwork.cs:165).  A recorded prad_adam_multi / prad_clip_adam_multi keeps
 *      its bias-correction factors as launch arguments; prad_graph_launch replaces them before each launch so that
 *      launch number k of a sequence recorded with AdamIteration t runs with t + k (k = 0, 1, ...), bit for bit what
 *      the eager calls with those iterations give.  prad_graph_set_adam_iteration sets the value the next launch
 *      uses (later launches continue from it). */
int32_t prad_graph_begin(void);
int32_t prad_graph_end(void** graph);
int32_t prad_graph_launch(void* graph);
int32_t prad_graph_set_adam_iteration(void* graph, double t);
int32_t prad_graph_destroy(void* graph);

/* Softmax.Forward (p), CategoricalCrossEntropy.Forward (loss, may be NULL) and .Backward (dp) and
 * Softmax.Backward (dx) of one batch; same arithmetic as prad_softmax_fwd + prad_cce_fwd + prad_cce_bwd +
 * prad_softmax_bwd (src/RMAD/SoftmaxOperation.cs:45-110,
 * src/RMAD/Loss/CategoricalCrossEntropyLossOperation.cs:37-86), in one launch. */
int32_t prad_softmax_cce(prad_buf_t x, prad_buf_t target, prad_buf_t p, prad_buf_t loss, prad_buf_t dp, prad_buf_t dx);

/* The output layer of a classifier with its loss, forward and backward: MatrixMultiplyOperation.Forward
 * (src/RMAD/MatrixMultiplyOperation.cs:50-80) and MatrixAddBroadcastingOperation.Forward into z, then everything
 * prad_softmax_cce does (p, loss, dp, dz), then the layer's Backward as prad_matmul_bias_bwd does it
 * (src/RMAD/MatrixMultiplyOperation.cs:94-126): dbias, dW (+)= A^T . dz, dA = dz . W^T times the derivative of the
 * activation below (act, act_src: what that activation cached, alpha) - the values of prad_matmul_fwd_fused +
 * prad_softmax_cce + prad_matmul_bias_bwd.  One launch of one workgroup when there are at most 64 classes, fewer than
 * 2048 rows and A, W and the class rows fit the compute unit's LDS (144 KB); the three launches otherwise.  bias, loss,
 * dbias and act_src (with act = PRAD_ACT_NONE) may be NULL. */
int32_t prad_dense_softmax_cce(prad_buf_t A, prad_buf_t W, prad_buf_t bias, prad_buf_t target, prad_buf_t z, prad_buf_t p,
                               prad_buf_t loss, prad_buf_t dp, prad_buf_t dz, prad_buf_t dA, prad_buf_t dW, prad_buf_t dbias,
                               int32_t accumulate_dW, int32_t act, prad_buf_t act_src, double alpha);

/* ---- GradientClipper.ClipGradients, src/RMAD/GradientClipper.cs:118-157 and :212-253 (in place) */
int32_t prad_clip(prad_buf_t g, double clip_value, double min_value);
/* ---- AdamOptimizer.UpdateWeightWithAdam, src/RMAD/AdamOptimizer.cs:195-239 (in place on w, m, v) */
int32_t prad_adam(prad_buf_t w, prad_buf_t m, prad_buf_t v, prad_buf_t g, double lr, double beta1, double beta2,
                  double eps, double t);
/* Multi-tensor forms: one launch sequence over n tensors (the Parallel.For over layers of
 * GradientClipper.Clip, src/RMAD/GradientClipper.cs:31-71, and AdamOptimizer.Optimize,
 * src/RMAD/AdamOptimizer.cs:32-91). */
int32_t prad_clip_multi(const prad_buf_t* g, int32_t n, double clip_value, double min_value);
int32_t prad_adam_multi(const prad_buf_t* w, const prad_buf_t* m, const prad_buf_t* v, const prad_buf_t* g, int32_t n,
                        double lr, double beta1, double beta2, double eps, double t);
/* AdamOptimizer.Revert -> ReverseAdamUpdate, src/RMAD/AdamOptimizer.cs:97-156 and :158-193: undoes the
 * update that produced the given w, m, v from the given gradient, statement for statement
 * (w += lr * mhat / (sqrt(vhat) + eps) from the current moments, then m = (m - (1 - beta1) g) / beta1,
 * v = (v - (1 - beta2) g g) / beta2).  t is the AdamIteration of the update being undone. */
int32_t prad_adam_revert_multi(const prad_buf_t* w, const prad_buf_t* m, const prad_buf_t* v, const prad_buf_t* g, int32_t n,
                               double lr, double beta1, double beta2, double eps, double t);
/* GradientClipper.Clip immediately followed by AdamOptimizer.Optimize over the same tensors, as every
 * training loop of the reference calls them
 * (examples/feedforward/ParallelReverseAutoDiff.FeedForwardExample/FeedForwardNeuralNetwork.cs:287-303): the clamping
 * pass and the update share one pass over the data.  Results (clamped g, w, m, v) are those of
 * prad_clip_multi followed by prad_adam_multi. */
int32_t prad_clip_adam_multi(const prad_buf_t* w, const prad_buf_t* m, const prad_buf_t* v, const prad_buf_t* g, int32_t n,
                             double clip_value, double min_value, double lr, double beta1, double beta2, double eps,
                             double t);

/* ---- allocation-free form of prad_clip_adam_multi.  No counterpart in the reference: it is for callers that cannot
 *      allocate at the point of the call (a launch sequence being captured, a tight serving or training loop, a
 *      harness that forbids hipMalloc).  Same arguments, same results (clamped g, w, m, v) bit for bit.  It never calls
 *      hipMalloc / hipFree and uses no host heap: the clip statistics go to a static device array of 1 MiB inside the
 *      library (one per GPU, held until the process ends) instead of the growable workspace.  Limits: at most 64
 *      tensors per call and at most about 43 000 chunks of 4096 elements in all (roughly 1.7e8 elements); beyond them
 *      it returns PRAD_ERR_ARG and enqueues nothing.  Every call on a GPU shares that array: calls that overlapped on
 *      one GPU would race, which the single library stream rules out for calls made through this library. */
int32_t prad_clip_adam_multi_noalloc(const prad_buf_t* w, const prad_buf_t* m, const prad_buf_t* v, const prad_buf_t* g, int32_t n,
                                     double clip_value, double min_value, double lr, double beta1, double beta2, double eps,
                                     double t);

/* ---- timing helpers for harnesses: events recorded on the library stream ------------------ */
int32_t prad_event_create(void** ev);
int32_t prad_event_destroy(void* ev);
int32_t prad_event_record(void* ev);
int32_t prad_event_elapsed_ms(void* start, void* stop, float* ms); /* waits for `stop` */

#ifdef __cplusplus
}
#endif
#endif /* PRAD_HIP_H */
