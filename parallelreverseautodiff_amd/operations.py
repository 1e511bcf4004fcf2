"""Operation classes with the reference's names and Forward/Backward contract, running on the
HIP library.

Boundary kept (src/RMAD/IOperation.cs:17-25, src/RMAD/Operation.cs:11-19,
src/RMAD/BackwardResult.cs, src/RMAD/BackwardResultBuilder.cs:27-63): a static
``Instantiate(net)``, a public ``Forward`` whose positional parameters are the graph inputs, a
``Backward(dOutput)`` that returns a ``BackwardResult`` whose ``Results`` are in input order,
``Store(id)`` / ``Restore(id)`` for per-sample intermediates, and ``GetOutput()``.

All four matrix-multiply names of the reference - MatrixMultiplyOperation
(src/RMAD/MatrixMultiplyOperation.cs), GpuMatrixMultiplyOperation
(src/RMAD/GpuMatrixMultiplyOperation.cs), CudaMatrixMultiplyOperation
(src/RMAD/CudaMatrixMultiplyOperation.cs) and GpuMatrixMultiplyAndSumOperation
(src/RMAD/GpuMatrixMultiplyAndSumOperation.cs) - resolve to the same device kernels; inputs and
outputs stay resident on the device between operations.
"""
import ctypes

import numpy as np

from . import _lib
from .cudablas import CudaBlas
from .exceptions import ArgumentException, CudaNotInitializedException, InvalidOperationException, check
from .matrix import DeepMatrix, DeviceBuffer, Matrix


class BackwardResult:
    """src/RMAD/BackwardResult.cs"""

    def __init__(self, results, has_multiple_inputs):
        self.Results = list(results)
        self.HasMultipleInputs = has_multiple_inputs

    @property
    def Item1(self):
        return self.Results[0]

    @property
    def Item2(self):
        return self.Results[1]

    @property
    def Item3(self):
        return self.Results[2]


class BackwardResultBuilder:
    """src/RMAD/BackwardResultBuilder.cs:27-63, :185-188"""

    def __init__(self):
        self._results = []
        self._input_gradients = 0

    def AddInputGradient(self, matrix):
        self._input_gradients += 1
        self._results.append(matrix)
        return self

    def AddInputGradientArray(self, deep):
        for m in deep:
            self.AddInputGradient(m)
        return self

    def AddBiasGradient(self, matrix):
        self._results.append(matrix)
        return self

    def Build(self):
        return BackwardResult(self._results, self._input_gradients > 1)


def _require_initialized():
    inst = CudaBlas.Instance
    if not inst.known_ready and not inst.IsInitialized:
        raise CudaNotInitializedException()


def _ensure_initialized():
    # MatrixMultiplyOperation has no initialisation requirement in the reference; starting the
    # device on first use keeps that.
    inst = CudaBlas.Instance
    if not inst.known_ready and not inst.IsInitialized:
        inst.Initialize()


def _null():
    return ctypes.c_void_p(None)


class Operation:
    """Common state of an operation node (src/RMAD/OperationBase.cs:261-264, IOperationBase.cs:188-194)."""

    def __init__(self):
        self.Output = None
        self._stored = {}

    def GetOutput(self):
        return self.Output

    def _intermediates(self):
        return []

    def _restore_from(self, items):
        pass

    def Store(self, id):
        self._stored[id] = self._intermediates()

    def Restore(self, id):
        self._restore_from(self._stored[id])


class MatrixMultiplyOperation(Operation):
    """C = A.B; Backward returns [dA = dC.B^T, dB = A^T.dC] (src/RMAD/MatrixMultiplyOperation.cs:50-126)."""

    _needs_init = False

    def __init__(self):
        super().__init__()
        self.input1 = None
        self.input2 = None

    @staticmethod
    def Instantiate(net):
        return MatrixMultiplyOperation()

    def _intermediates(self):
        return [self.input1, self.input2]

    def _restore_from(self, items):
        self.input1, self.input2 = items

    def _check_device(self):
        if self._needs_init:
            _require_initialized()
        else:
            _ensure_initialized()

    def Forward(self, input1, input2):
        self._check_device()
        self.input1, self.input2 = input1, input2
        if input1.Cols != input2.Rows:
            raise InvalidOperationException("Input 1 columns do not match Input 2 rows")
        if input1.dtype != input2.dtype:
            raise ArgumentException("buffers of different element types in one call")
        out = DeviceBuffer.alloc_output(input1.dtype, input1.Rows, input2.Cols)
        check(_lib.load().prad_matmul_fwd(input1.device().handle, input2.device().handle, out.handle))
        self.Output = Matrix._from_device(out)
        return self.Output

    def Backward(self, dOutput):
        self._check_device()
        a, b = self.input1, self.input2
        d_in1 = DeviceBuffer.alloc_output(a.dtype, a.Rows, a.Cols)
        d_in2 = DeviceBuffer.alloc_output(b.dtype, b.Rows, b.Cols)
        check(_lib.load().prad_matmul_bwd(dOutput.device().handle, a.device().handle, b.device().handle,
                                         d_in1.handle, d_in2.handle, 0, 0))
        return (BackwardResultBuilder()
                .AddInputGradient(Matrix._from_device(d_in1))
                .AddInputGradient(Matrix._from_device(d_in2))
                .Build())


class GpuMatrixMultiplyOperation(MatrixMultiplyOperation):
    """Same contract; requires CudaBlas.Instance.Initialize() first (src/RMAD/GpuMatrixMultiplyOperation.cs:113-161)."""

    _needs_init = True

    @staticmethod
    def Instantiate(net):
        return GpuMatrixMultiplyOperation()


class CudaMatrixMultiplyOperation(MatrixMultiplyOperation):
    """Same contract (src/RMAD/CudaMatrixMultiplyOperation.cs:51-96)."""

    _needs_init = True

    @staticmethod
    def Instantiate(net):
        return CudaMatrixMultiplyOperation()


class _BatchMatrixMultiplyBase(Operation):
    """Per-sample products over a DeepMatrix as one strided-batched launch
    (src/RMAD/BatchGpuMatrixMultiplyOperation.cs:56-143, BatchMatrixMultiplyOperation.cs:51-94)."""

    _needs_init = True

    def __init__(self):
        super().__init__()
        self.DeepOutput = None
        self._in1 = None
        self._in2 = None

    def GetDeepOutput(self):
        return self.DeepOutput

    def Forward(self, input1, input2):
        if self._needs_init:
            _require_initialized()
        else:
            _ensure_initialized()
        deep1, deep2 = isinstance(input1, DeepMatrix), isinstance(input2, DeepMatrix)
        if not (deep1 or deep2):
            raise ArgumentException("at least one input must be a DeepMatrix")
        depth = input1.Depth if deep1 else input2.Depth
        if deep1 and deep2 and input1.Depth != input2.Depth:
            raise ArgumentException("inputs of different depth")
        if input1.Cols != input2.Rows:
            raise InvalidOperationException("Input 1 columns do not match Input 2 rows")
        self._in1, self._in2 = input1, input2
        out = DeviceBuffer.alloc_output(input1.dtype, input1.Rows, input2.Cols, depth=depth)
        check(_lib.load().prad_gemm_batched(0, 0, input1.device().handle, input2.device().handle, out.handle, 0))
        self.DeepOutput = DeepMatrix._from_device(out)
        return self.DeepOutput

    def Backward(self, dOutput):
        if self._needs_init:
            _require_initialized()
        lib = _lib.load()
        depth = dOutput.Depth
        a, b = self._in1, self._in2
        d1 = DeviceBuffer.alloc_output(a.dtype, a.Rows, a.Cols, depth=depth)
        d2 = DeviceBuffer.alloc_output(b.dtype, b.Rows, b.Cols, depth=depth)
        g = dOutput.device()
        check(lib.prad_gemm_batched(0, 1, g.handle, b.device().handle, d1.handle, 0))  # dA_i = dC_i . B_i^T
        check(lib.prad_gemm_batched(1, 0, a.device().handle, g.handle, d2.handle, 0))  # dB_i = A_i^T . dC_i
        m1, m2 = DeepMatrix._from_device(d1), DeepMatrix._from_device(d2)
        return [BackwardResultBuilder().AddInputGradient(m1[i]).AddInputGradient(m2[i]).Build() for i in range(depth)]


class BatchMatrixMultiplyOperation(_BatchMatrixMultiplyBase):
    _needs_init = False

    @staticmethod
    def Instantiate(net):
        return BatchMatrixMultiplyOperation()


class BatchGpuMatrixMultiplyOperation(_BatchMatrixMultiplyBase):
    @staticmethod
    def Instantiate(net):
        return BatchGpuMatrixMultiplyOperation()


class BatchCudaMatrixMultiplyOperation(_BatchMatrixMultiplyBase):
    @staticmethod
    def Instantiate(net):
        return BatchCudaMatrixMultiplyOperation()


class MatrixMultiplyAndSumOperation(Operation):
    """out[0][q] = sum_ij (A.B[q])_ij; Backward as the reference writes it
    (src/RMAD/MatrixMultiplyAndSumOperation.cs:50-89)."""

    _needs_init = False

    def __init__(self):
        super().__init__()
        self.a = None
        self.b = None

    @staticmethod
    def Instantiate(net):
        return MatrixMultiplyAndSumOperation()

    def _intermediates(self):
        return [self.a, self.b]

    def _restore_from(self, items):
        self.a, self.b = items

    def Forward(self, a, b):
        if self._needs_init:
            _require_initialized()
        else:
            _ensure_initialized()
        self.a, self.b = a, b
        if a.Cols != b.Rows:
            raise InvalidOperationException("Matrix dimensions must be compatible for multiplication.")
        out = DeviceBuffer.alloc_output(a.dtype, 1, b.Depth)
        check(_lib.load().prad_matmul_sum_fwd(a.device().handle, b.device().handle, out.handle))
        self.Output = Matrix._from_device(out)
        return self.Output

    def Backward(self, dOutput):
        if self._needs_init:
            _require_initialized()
        a, b = self.a, self.b
        d_a = DeviceBuffer.alloc_output(a.dtype, a.Rows, a.Cols)
        d_b = DeviceBuffer.alloc_output(a.dtype, a.Cols, a.Rows, depth=b.Depth)
        check(_lib.load().prad_matmul_sum_bwd(a.device().handle, b.device().handle, dOutput.device().handle,
                                             d_a.handle, d_b.handle))
        return (BackwardResultBuilder()
                .AddInputGradient(Matrix._from_device(d_a))
                .AddInputGradientArray(DeepMatrix._from_device(d_b))
                .Build())


class GpuMatrixMultiplyAndSumOperation(MatrixMultiplyAndSumOperation):
    """src/RMAD/GpuMatrixMultiplyAndSumOperation.cs:114-154"""

    _needs_init = True

    @staticmethod
    def Instantiate(net):
        return GpuMatrixMultiplyAndSumOperation()


class _BatchMatrixMultiplyAndSumBase(Operation):
    """MatrixMultiplyAndSum per sample of a batch (src/RMAD/BatchGpuMatrixMultiplyAndSumOperation.cs:51-74,
    src/RMAD/BatchMatrixMultiplyAndSumOperation.cs:51-74): Forward(input1 deep of S samples, input2 deep of P slices)
    returns a DeepMatrix of S matrices 1 x P, sample i being MatrixMultiplyAndSum(input1[i], input2); Backward(dOutput
    deep of S matrices 1 x P) returns one BackwardResult per sample, [dA_i, dB_i[0], ..., dB_i[P-1]] as the single
    operation builds it.  The reference loops over the samples (Parallel.For in Backward); here every sample and
    slice shares one launch each way."""

    _needs_init = True

    def __init__(self):
        super().__init__()
        self.DeepOutput = None
        self._in1 = None
        self._in2 = None

    def GetDeepOutput(self):
        return self.DeepOutput

    def _intermediates(self):
        return [self._in1, self._in2]

    def _restore_from(self, items):
        self._in1, self._in2 = items

    def Forward(self, input1, input2):
        if self._needs_init:
            _require_initialized()
        else:
            _ensure_initialized()
        if not isinstance(input1, DeepMatrix) or not isinstance(input2, DeepMatrix):
            raise ArgumentException("both inputs must be DeepMatrix")
        if input1.Cols != input2.Rows:
            raise InvalidOperationException("Matrix dimensions must be compatible for multiplication.")
        self._in1, self._in2 = input1, input2
        out = DeviceBuffer.alloc_output(input1.dtype, 1, input2.Depth, depth=input1.Depth)
        check(_lib.load().prad_matmul_sum_fwd(input1.device().handle, input2.device().handle, out.handle))
        self.DeepOutput = DeepMatrix._from_device(out)
        return self.DeepOutput

    def Backward(self, dOutput):
        if self._needs_init:
            _require_initialized()
        a, b = self._in1, self._in2
        S, P = a.Depth, b.Depth
        if dOutput.Depth != S:
            raise ArgumentException("upstream gradient must hold one matrix per sample")
        d_a = DeviceBuffer.alloc_output(a.dtype, a.Rows, a.Cols, depth=S)
        d_b = DeviceBuffer.alloc_output(a.dtype, a.Cols, a.Rows, depth=S * P)
        check(_lib.load().prad_matmul_sum_bwd(a.device().handle, b.device().handle, dOutput.device().handle, d_a.handle, d_b.handle))
        m_a, m_b = DeepMatrix._from_device(d_a), DeepMatrix._from_device(d_b)
        return [BackwardResultBuilder().AddInputGradient(m_a[i]).AddInputGradientArray([m_b[i * P + q] for q in range(P)]).Build()
                for i in range(S)]


class BatchMatrixMultiplyAndSumOperation(_BatchMatrixMultiplyAndSumBase):
    _needs_init = False

    @staticmethod
    def Instantiate(net):
        return BatchMatrixMultiplyAndSumOperation()


class BatchGpuMatrixMultiplyAndSumOperation(_BatchMatrixMultiplyAndSumBase):
    @staticmethod
    def Instantiate(net):
        return BatchGpuMatrixMultiplyAndSumOperation()


class BatchMatrixMultiplySumOperation(Operation):
    """Independent products summed into one output plus a broadcast bias: C = sum_q A[q].B[q] + bias.
    No operation of the reference has this form; it is the composition of MatrixMultiplyOperation.Forward
    per slice (src/RMAD/MatrixMultiplyOperation.cs:50-80), a sum of the products in slice order and
    MatrixAddBroadcastingOperation (src/RMAD/MatrixAddBroadcastingOperation.cs:32-70), run as one split
    product.  Backward returns [dA (deep), dB (deep), dBias]."""

    def __init__(self):
        super().__init__()
        self.a = self.b = self.bias = None

    @staticmethod
    def Instantiate(net):
        return BatchMatrixMultiplySumOperation()

    def _intermediates(self):
        return [self.a, self.b, self.bias]

    def _restore_from(self, items):
        self.a, self.b, self.bias = items

    def Forward(self, a, b, bias=None):
        _ensure_initialized()
        self.a, self.b, self.bias = a, b, bias
        if a.Cols != b.Rows:
            raise InvalidOperationException("Input 1 columns do not match Input 2 rows")
        out = DeviceBuffer.alloc_output(a.dtype, a.Rows, b.Cols)
        check(_lib.load().prad_matmul_batch_sum_fwd(a.device().handle, b.device().handle,
                                                   None if bias is None else bias.device().handle, out.handle))
        self.Output = Matrix._from_device(out)
        return self.Output

    def Backward(self, dOutput):
        a, b = self.a, self.b
        d_a = DeviceBuffer.alloc_output(a.dtype, a.Rows, a.Cols, depth=a.Depth)
        d_b = DeviceBuffer.alloc_output(a.dtype, b.Rows, b.Cols, depth=b.Depth)
        d_bias = None if self.bias is None else DeviceBuffer.alloc_output(a.dtype, 1, b.Cols)
        check(_lib.load().prad_matmul_batch_sum_bwd(dOutput.device().handle, a.device().handle, b.device().handle, d_a.handle,
                                                   d_b.handle, None if d_bias is None else d_bias.handle))
        builder = BackwardResultBuilder().AddInputGradient(DeepMatrix._from_device(d_a)).AddInputGradient(DeepMatrix._from_device(d_b))
        if d_bias is not None:
            builder.AddBiasGradient(Matrix._from_device(d_bias))
        return builder.Build()


class _ActivationOperation(Operation):
    """Elementwise activation; ``_caches`` says whether Backward needs the input or the output."""

    _act = _lib.ACT_NONE
    _caches = "input"

    def __init__(self, alpha=0.0):
        super().__init__()
        self.alpha = alpha
        self.input = None

    def _intermediates(self):
        return [self.input, self.Output]

    def _restore_from(self, items):
        self.input, self.Output = items

    def Forward(self, input):
        _ensure_initialized()
        self.input = input
        out = DeviceBuffer.alloc_output(input.dtype, input.Rows, input.Cols)
        check(_lib.load().prad_act_fwd(self._act, input.device().handle, out.handle, float(self.alpha)))
        self.Output = Matrix._from_device(out)
        return self.Output

    def Backward(self, dOutput):
        _ensure_initialized()
        src = self.input if self._caches == "input" else self.Output
        dx = DeviceBuffer.alloc_output(src.dtype, src.Rows, src.Cols)
        check(_lib.load().prad_act_bwd(self._act, src.device().handle, dOutput.device().handle, dx.handle, float(self.alpha)))
        return BackwardResultBuilder().AddInputGradient(Matrix._from_device(dx)).Build()


class LeakyReLUOperation(_ActivationOperation):
    """src/RMAD/LeakyReLUOperation.cs:54-93; alpha comes from net.Parameters.LeakyReLUAlpha (:32-35)."""

    _act = _lib.ACT_LEAKYRELU

    def __init__(self, alpha=0.01):
        super().__init__(alpha)

    @staticmethod
    def Instantiate(net):
        params = getattr(net, "Parameters", None)
        return LeakyReLUOperation(getattr(params, "LeakyReLUAlpha", 0.01))


class SigmoidOperation(_ActivationOperation):
    """src/RMAD/SigmoidOperation.cs:46-84"""

    _act = _lib.ACT_SIGMOID
    _caches = "output"

    @staticmethod
    def Instantiate(net):
        return SigmoidOperation()


class TanhOperation(_ActivationOperation):
    """src/RMAD/TanhOperation.cs:42-79"""

    _act = _lib.ACT_TANH
    _caches = "output"

    @staticmethod
    def Instantiate(net):
        return TanhOperation()


class GELUOperation(_ActivationOperation):
    """src/RMAD/GELUOperation.cs:44-101 (Backward uses the reference's own derivative formula)."""

    _act = _lib.ACT_GELU

    @staticmethod
    def Instantiate(net):
        return GELUOperation()


class HadamardProductOperation(Operation):
    """src/RMAD/HadamardProductOperation.cs:50-118"""

    def __init__(self):
        super().__init__()
        self.input1 = None
        self.input2 = None

    @staticmethod
    def Instantiate(net):
        return HadamardProductOperation()

    def _intermediates(self):
        return [self.input1, self.input2]

    def _restore_from(self, items):
        self.input1, self.input2 = items

    def Forward(self, input1, input2):
        _ensure_initialized()
        self.input1, self.input2 = input1, input2
        if input1.Rows != input2.Rows or input1.Cols != input2.Cols:
            raise ArgumentException("Matrices must have the same dimensions.")
        out = DeviceBuffer.alloc_output(input1.dtype, input1.Rows, input1.Cols)
        check(_lib.load().prad_hadamard_fwd(input1.device().handle, input2.device().handle, out.handle))
        self.Output = Matrix._from_device(out)
        return self.Output

    def Backward(self, dOutput):
        _ensure_initialized()
        a, b = self.input1, self.input2
        da = DeviceBuffer.alloc_output(a.dtype, a.Rows, a.Cols)
        db = DeviceBuffer.alloc_output(a.dtype, a.Rows, a.Cols)
        check(_lib.load().prad_hadamard_bwd(a.device().handle, b.device().handle, dOutput.device().handle, da.handle, db.handle))
        return (BackwardResultBuilder()
                .AddInputGradient(Matrix._from_device(da))
                .AddInputGradient(Matrix._from_device(db))
                .Build())


class AmplifiedSigmoidOperation(_ActivationOperation):
    """src/RMAD/AmplifiedSigmoidOperation.cs:44-84: 1 / (1 + pow(PI - 2, -x)); Backward as written there."""

    _act = _lib.ACT_AMPLIFIED_SIGMOID

    @staticmethod
    def Instantiate(net):
        return AmplifiedSigmoidOperation()


class MatrixAddOperation(Operation):
    """y = a + b; Backward returns two copies of dOutput (src/RMAD/MatrixAddOperation.cs:30-68).  The copies are
    the upstream gradient itself here: nothing writes into a gradient it received."""

    @staticmethod
    def Instantiate(net):
        return MatrixAddOperation()

    def Forward(self, inputA, inputB):
        _ensure_initialized()
        out = DeviceBuffer.alloc_output(inputA.dtype, inputA.Rows, inputA.Cols)
        check(_lib.load().prad_add(inputA.device().handle, inputB.device().handle, out.handle))
        self.Output = Matrix._from_device(out)
        return self.Output

    def Backward(self, dOutput):
        return BackwardResultBuilder().AddInputGradient(dOutput).AddInputGradient(dOutput).Build()


class MatrixAddThreeOperation(Operation):
    """y = a + b + bias; Backward returns dOutput for a, b and as the bias gradient
    (src/RMAD/MatrixAddThreeOperation.cs:35-70)."""

    @staticmethod
    def Instantiate(net):
        return MatrixAddThreeOperation()

    def Forward(self, inputA, inputB, bias):
        _ensure_initialized()
        out = DeviceBuffer.alloc_output(inputA.dtype, inputA.Rows, inputA.Cols)
        check(_lib.load().prad_add_three(inputA.device().handle, inputB.device().handle, bias.device().handle, out.handle))
        self.Output = Matrix._from_device(out)
        return self.Output

    def Backward(self, dOutput):
        return BackwardResultBuilder().AddInputGradient(dOutput).AddInputGradient(dOutput).AddBiasGradient(dOutput).Build()


class MatrixTransposeOperation(Operation):
    """src/RMAD/MatrixTransposeOperation.cs:30-64"""

    @staticmethod
    def Instantiate(net):
        return MatrixTransposeOperation()

    @staticmethod
    def _transpose(m):
        _ensure_initialized()
        out = DeviceBuffer.alloc_output(m.dtype, m.Cols, m.Rows)
        check(_lib.load().prad_transpose(m.device().handle, out.handle))
        return Matrix._from_device(out)

    def Forward(self, input):
        self.Output = self._transpose(input)
        return self.Output

    def Backward(self, dOutput):
        return BackwardResultBuilder().AddInputGradient(self._transpose(dOutput)).Build()


class LayerNormalizationOperation(Operation):
    """src/RMAD/LayerNormalizationOperation.cs:56-110: row-wise (x - mean) / (stddev + 1e-9); caches the input and
    the per-row mean and deviation (device buffers here); Backward as written in the reference."""

    def __init__(self):
        super().__init__()
        self.input = self.mean = self.stdDev = None

    @staticmethod
    def Instantiate(net):
        return LayerNormalizationOperation()

    def _intermediates(self):
        return [self.input, self.mean, self.stdDev]

    def _restore_from(self, items):
        self.input, self.mean, self.stdDev = items

    def Forward(self, input):
        _ensure_initialized()
        self.input = input
        out = DeviceBuffer.alloc_output(input.dtype, input.Rows, input.Cols)
        self.mean = DeviceBuffer.alloc_output(input.dtype, 1, input.Rows)
        self.stdDev = DeviceBuffer.alloc_output(input.dtype, 1, input.Rows)
        check(_lib.load().prad_layernorm_fwd(input.device().handle, out.handle, self.mean.handle, self.stdDev.handle))
        self.Output = Matrix._from_device(out)
        return self.Output

    def Backward(self, gradOutput):
        _ensure_initialized()
        dx = DeviceBuffer.alloc_output(self.input.dtype, self.input.Rows, self.input.Cols)
        check(_lib.load().prad_layernorm_bwd(self.input.device().handle, self.mean.handle, self.stdDev.handle,
                                             gradOutput.device().handle, dx.handle))
        return BackwardResultBuilder().AddInputGradient(Matrix._from_device(dx)).Build()


class MatrixAddBroadcastingOperation(Operation):
    """y = x + bias (1 x N); Backward returns [dOutput itself, dBias] with HasMultipleInputs false
    (src/RMAD/MatrixAddBroadcastingOperation.cs:32-70)."""

    @staticmethod
    def Instantiate(net):
        return MatrixAddBroadcastingOperation()

    def Forward(self, input, bias):
        _ensure_initialized()
        if input.Cols != bias.Cols:
            raise ArgumentException(
                "The length of the bias vector must be the same as the number of columns in the input matrix.")
        out = DeviceBuffer.alloc_output(input.dtype, input.Rows, input.Cols)
        check(_lib.load().prad_add_broadcast_fwd(input.device().handle, bias.device().handle, out.handle))
        self.Output = Matrix._from_device(out)
        return self.Output

    def Backward(self, dOutput):
        _ensure_initialized()
        db = DeviceBuffer.alloc_output(dOutput.dtype, 1, dOutput.Cols)
        check(_lib.load().prad_add_broadcast_bwd_bias(dOutput.device().handle, db.handle))
        return BackwardResultBuilder().AddInputGradient(dOutput).AddBiasGradient(Matrix._from_device(db)).Build()


def accumulate_gradient(dest, grad):
    """dest[i][j] += grad[i][j] on the device (OperationBase.AccumulateGradient, src/RMAD/OperationBase.cs:295-303)."""
    _ensure_initialized()
    if dest.Rows != grad.Rows or dest.Cols != grad.Cols:
        raise ArgumentException("Matrices must have the same dimensions.")
    check(_lib.load().prad_accumulate(dest.device().handle, grad.device().handle))
    dest._device_written()


def handle_array(buffers):
    """ctypes array of prad_buf_t for the multi-tensor entry points."""
    return (ctypes.c_void_p * len(buffers))(*[b.handle.value for b in buffers])


class SoftmaxOperation(Operation):
    """Row-wise softmax (src/RMAD/SoftmaxOperation.cs:45-110)."""

    @staticmethod
    def Instantiate(net):
        return SoftmaxOperation()

    def Forward(self, input):
        _ensure_initialized()
        out = DeviceBuffer.alloc_output(input.dtype, input.Rows, input.Cols)
        check(_lib.load().prad_softmax_fwd(input.device().handle, out.handle))
        self.Output = Matrix._from_device(out)
        return self.Output

    def Backward(self, dLdOutput):
        _ensure_initialized()
        y = self.Output
        dx = DeviceBuffer.alloc_output(y.dtype, y.Rows, y.Cols)
        check(_lib.load().prad_softmax_bwd(y.device().handle, dLdOutput.device().handle, dx.handle))
        return BackwardResultBuilder().AddInputGradient(Matrix._from_device(dx)).Build()


class CategoricalCrossEntropyLossOperation(Operation):
    """loss = sum(-t log(p + 1e-15)) / rows (src/RMAD/Loss/CategoricalCrossEntropyLossOperation.cs:37-86)."""

    def __init__(self):
        super().__init__()
        self.target = None

    @staticmethod
    def Instantiate(net):
        return CategoricalCrossEntropyLossOperation()

    def Forward(self, output, target):
        _ensure_initialized()
        if target is None:
            raise ArgumentException("target")
        if output.Rows != target.Rows or output.Cols != target.Cols:
            raise ArgumentException("Output and target matrices must have the same dimensions.")
        self.target = target
        loss = DeviceBuffer.alloc_output(output.dtype, 1, 1)
        check(_lib.load().prad_cce_fwd(output.device().handle, target.device().handle, loss.handle))
        self.Output = Matrix._from_device(loss)
        return self.Output

    def Backward(self, output):
        _ensure_initialized()
        dp = DeviceBuffer.alloc_output(output.dtype, output.Rows, output.Cols)
        check(_lib.load().prad_cce_bwd(output.device().handle, self.target.device().handle, dp.handle))
        return BackwardResultBuilder().AddInputGradient(Matrix._from_device(dp)).Build()
