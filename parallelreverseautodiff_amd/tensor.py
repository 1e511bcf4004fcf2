"""The tape engine's tensor product on the device: Tensor.MatrixMultiply (src/PRAD/Tensor.cs:572-608) and
TensorReverse.MatrixMultiplyReverse (src/PRAD/TensorReverse.cs:94-157).

The reference Tensor is a shape plus one flat row-major ``double[]`` (``float[]`` in PRADLite) that it hands to
a BLAS gemm.  Here the flat array has a device twin (a dense buffer of libprad_hip): products read and write
the device copy, the host array is filled when ``Data`` is read.  A flat array crosses the boundary as one
strided copy, without the per-row marshalling the jagged Matrix needs.

Beyond two dimensions.  The reference's method throws for anything but 2-D operands (Tensor.cs:574-577), while its
own windowed-attention example multiplies 3-D and 4-D tensors (examples/swin/SwinExample/SwinTransformerTools.cs:348-399:
``[windows, tokens, C] . [C, 3C]``, ``[windows, heads, tokens, d] . [windows, heads, d, tokens]``) and so cannot run as
written.  Here the product is defined on the last two dimensions, as that example needs it:

  * ``[..., m, k] . [..., k, n]`` with equal leading dimensions: one product per leading index (one strided-batched
    launch); gradients per slice, ``dA = dC . B^T`` and ``dB = A^T . dC``;
  * ``[..., m, k] . [k, n]``: the right operand is shared; the left one is a (prod(...) * m) x k matrix as it lies in
    memory, so this is one plain product, and ``dB = A^T . dC`` over all leading indices is one product too.

Two 2-D operands behave exactly as in the reference, error messages included.
"""
import ctypes

import numpy as np

from . import _lib
from .exceptions import ArgumentException, InvalidOperationException, check
from .matrix import DeviceBuffer, _dtype_code
from .operations import _ensure_initialized

_MAX_BATCH = 65535  # products per strided-batched launch


class Tensor:
    def __init__(self, shape, data=None, dtype=np.float64):
        self.Shape = [int(s) for s in shape]
        self.dtype = np.dtype(dtype if data is None or not hasattr(data, "dtype") else data.dtype)
        count = int(np.prod(self.Shape)) if self.Shape else 1
        self._dev = None
        if data is None:
            self._host = np.zeros(count, self.dtype)
        else:
            self._host = np.ascontiguousarray(data, dtype=self.dtype).reshape(-1)
            if self._host.size != count:
                raise ArgumentException("Data length does not match shape.")

    @classmethod
    def _from_device(cls, buf, shape=None):
        t = cls.__new__(cls)
        t.Shape = list(shape) if shape is not None else [buf.rows, buf.cols]
        t.dtype, t._dev, t._host = buf.dtype, buf, None
        return t

    @property
    def Data(self):
        """The flat row-major array (downloaded on first read after a device product).  The caller may write
        into it, as callers of the reference do, so the device copy is dropped."""
        if self._host is None:
            self._host = self._dev.download().reshape(-1)
        self._dev = None
        return self._host

    def to_numpy(self):
        flat = self._host if self._host is not None else self._dev.download().reshape(-1)
        return flat.reshape(self.Shape)

    # ---- device twin: a deep buffer of prod(leading dimensions) slices of the last two dimensions -------------------
    def _lead(self):
        return int(np.prod(self.Shape[:-2])) if len(self.Shape) > 2 else 1

    def _device(self):
        if self._dev is None:
            rows, cols = self.Shape[-2], self.Shape[-1]
            self._dev = DeviceBuffer.alloc(self.dtype, rows, cols, depth=self._lead())
            self._dev.upload(self._host.reshape(self._lead() * rows, cols))
        return self._dev

    def _flat_view(self):
        """The same device memory as one (prod(leading) * rows) x cols matrix."""
        dev = self._device()
        if dev.depth == 1:
            return dev
        h = ctypes.c_void_p()
        check(_lib.load().prad_buf_wrap(_dtype_code(self.dtype), dev.depth * dev.rows, dev.cols, ctypes.c_void_p(dev.ptr), ctypes.byref(h)))
        return DeviceBuffer(h, self.dtype, 1, dev.depth * dev.rows, dev.cols, parent=dev)

    def MatrixMultiply(self, other, alpha=1.0, beta=0.0):
        """alpha * this . other for two-dimensional tensors; anything else raises the reference's ArgumentException
        (src/PRAD/Tensor.cs:574-577).  ``beta`` multiplies the freshly zeroed result array in the reference and has no
        effect; it is accepted for signature compatibility."""
        if len(self.Shape) != 2 or len(other.Shape) != 2:
            raise ArgumentException("Matrix multiplication is only supported for 2D tensors.")
        return self.BatchMatrixMultiply(other, alpha)

    def BatchMatrixMultiply(self, other, alpha=1.0):
        """alpha * this . other on the last two dimensions of tensors of two or more dimensions: one product per
        leading index ([..., m, k] . [..., k, n]), or a shared two-dimensional right operand ([..., m, k] . [k, n]).
        The reference has no such method (its MatrixMultiply rejects these shapes); it is what its windowed-attention
        example needs (examples/swin/SwinExample/SwinTransformerTools.cs:348-389)."""
        kind = _product_kind(self.Shape, other.Shape, "Matrix multiplication is only supported for 2D tensors.")
        if self.dtype != other.dtype:
            raise ArgumentException("buffers of different element types in one call")
        m, k, n = self.Shape[-2], self.Shape[-1], other.Shape[-1]
        _ensure_initialized()
        lib = _lib.load()
        if kind == "shared":
            a = self._flat_view()
            out = DeviceBuffer.alloc(self.dtype, a.rows, n)
            check(lib.prad_matmul_fwd(a.handle, other._device().handle, out.handle))
            out = _as_deep(out, self._lead(), m, n)
        else:
            lead = self._lead()
            out = DeviceBuffer.alloc(self.dtype, m, n, depth=lead)
            _batched(lib, 0, 0, self._device(), other._device(), out, m, n, k)
        if alpha != 1.0:
            check(lib.prad_scale(out.handle, out.handle, float(alpha)))
        return Tensor._from_device(out, self.Shape[:-1] + [n])


def _product_kind(shape_a, shape_b, message_2d):
    """'shared' (N-D . 2-D, which includes 2-D . 2-D: the left operand is one matrix as it lies in memory) or 'batched'
    (equal leading dimensions); raises the reference's exceptions for operands that do not multiply."""
    if len(shape_a) < 2 or len(shape_b) < 2:
        raise ArgumentException(message_2d)
    if shape_a[-1] != shape_b[-2]:
        raise ArgumentException("Incompatible shapes for matrix multiplication.")
    if len(shape_b) == 2 or all(d == 1 for d in shape_b[:-2]):
        return "shared"
    if list(shape_a[:-2]) != list(shape_b[:-2]):
        raise ArgumentException("Incompatible shapes for matrix multiplication.")
    return "batched"


def _as_deep(flat, lead, rows, cols):
    """A (lead * rows) x cols buffer seen as lead slices of rows x cols (same memory)."""
    if lead == 1:
        return flat
    h = ctypes.c_void_p()
    check(_lib.load().prad_buf_wrap_deep(_dtype_code(flat.dtype), lead, rows, cols, ctypes.c_void_p(flat.ptr), ctypes.byref(h)))
    return DeviceBuffer(h, flat.dtype, lead, rows, cols, parent=flat)


def _batched(lib, tA, tB, A, B, C, M, N, K):
    """C[s] = op(A[s]) . op(B[s]) for every slice s, in launches of at most 65535 products."""
    fn = lib.prad_gemm_strided_batched_f64 if C.dtype == np.float64 else lib.prad_gemm_strided_batched_f32
    es = C.dtype.itemsize
    sa, sb, sc = A.rows * A.cols, B.rows * B.cols, C.rows * C.cols
    lead = C.depth
    for s0 in range(0, lead, _MAX_BATCH):
        nb = min(_MAX_BATCH, lead - s0)
        check(fn(tA, tB, M, N, K, ctypes.c_void_p(A.ptr + s0 * sa * es), A.cols, sa, ctypes.c_void_p(B.ptr + s0 * sb * es), B.cols, sb,
                 ctypes.c_void_p(C.ptr + s0 * sc * es), C.cols, sc, nb, 0))


class TensorReverse:
    """src/PRAD/TensorReverse.cs: holds the tensors an operation consumed and computes their gradients."""

    def __init__(self, tensors):
        self.InitialTensors = list(tensors)

    def MatrixMultiplyReverse(self, upstreamGradient):
        """[dA, dB] for C = A . B of two-dimensional tensors: dA = dC . B^T and dB = A^T . dC
        (src/PRAD/TensorReverse.cs:94-157, which rejects other shapes)."""
        if len(self.InitialTensors) != 2:
            raise InvalidOperationException("MatrixMultiplyReverse expects exactly two initial tensors.")
        if any(len(t.Shape) != 2 for t in self.InitialTensors) or len(upstreamGradient.Shape) != 2:
            raise ArgumentException("Matrix multiplication gradients are only supported for 2D tensors.")
        return self.BatchMatrixMultiplyReverse(upstreamGradient)

    def BatchMatrixMultiplyReverse(self, upstreamGradient):
        """The gradients of BatchMatrixMultiply on the last two dimensions (per slice for a batched product; for a
        shared right operand dB adds up over all leading indices, which is the single product of the flattened
        operands)."""
        if len(self.InitialTensors) != 2:
            raise InvalidOperationException("MatrixMultiplyReverse expects exactly two initial tensors.")
        a, b = self.InitialTensors
        kind = _product_kind(a.Shape, b.Shape, "Matrix multiplication gradients are only supported for 2D tensors.")
        m, k, n = a.Shape[-2], a.Shape[-1], b.Shape[-1]
        if list(upstreamGradient.Shape) != list(a.Shape[:-1]) + [n]:
            raise ArgumentException("Incompatible shapes for matrix multiplication.")
        _ensure_initialized()
        lib = _lib.load()
        lead = a._lead()
        if kind == "shared":
            g, af = upstreamGradient._flat_view(), a._flat_view()
            d_a = DeviceBuffer.alloc(a.dtype, af.rows, k)
            d_b = DeviceBuffer.alloc(a.dtype, k, n)
            check(lib.prad_matmul_bwd(g.handle, af.handle, b._device().handle, d_a.handle, d_b.handle, 0, 0))
            return [Tensor._from_device(_as_deep(d_a, lead, m, k), a.Shape), Tensor._from_device(d_b, b.Shape)]
        d_a, d_b = DeviceBuffer.alloc(a.dtype, m, k, depth=lead), DeviceBuffer.alloc(a.dtype, k, n, depth=lead)
        g = upstreamGradient._device()
        _batched(lib, 0, 1, g, b._device(), d_a, m, k, n)   # dA[s] = dC[s] . B[s]^T
        _batched(lib, 1, 0, a._device(), g, d_b, k, n, m)   # dB[s] = A[s]^T . dC[s]
        return [Tensor._from_device(d_a, a.Shape), Tensor._from_device(d_b, b.Shape)]
