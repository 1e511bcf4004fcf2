"""The tape engine's tensor product on the device: Tensor.MatrixMultiply (src/PRAD/Tensor.cs:572-608) and
TensorReverse.MatrixMultiplyReverse (src/PRAD/TensorReverse.cs:94-157).

The reference Tensor is a shape plus one flat row-major ``double[]`` (``float[]`` in PRADLite) that it hands to
a BLAS gemm.  Here the flat array has a device twin (a dense buffer of libprad_hip): products read and write
the device copy, the host array is filled when ``Data`` is read.  A flat array crosses the boundary as one
strided copy, without the per-row marshalling the jagged Matrix needs.
"""
import numpy as np

from . import _lib
from .exceptions import ArgumentException, InvalidOperationException, check
from .matrix import DeviceBuffer
from .operations import _ensure_initialized


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
    def _from_device(cls, buf):
        t = cls.__new__(cls)
        t.Shape, t.dtype, t._dev, t._host = [buf.rows, buf.cols], buf.dtype, buf, None
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

    def _device(self):
        if self._dev is None:
            self._dev = DeviceBuffer.alloc(self.dtype, self.Shape[0], self.Shape[1])
            self._dev.upload(self._host.reshape(self.Shape))
        return self._dev

    def MatrixMultiply(self, other, alpha=1.0, beta=0.0):
        """alpha * this . other.  ``beta`` multiplies the freshly zeroed result array in the reference and has no
        effect; it is accepted for signature compatibility."""
        if len(self.Shape) != 2 or len(other.Shape) != 2:
            raise ArgumentException("Matrix multiplication is only supported for 2D tensors.")
        m, k, n = self.Shape[0], self.Shape[1], other.Shape[1]
        if k != other.Shape[0]:
            raise ArgumentException("Incompatible shapes for matrix multiplication.")
        _ensure_initialized()
        lib = _lib.load()
        out = DeviceBuffer.alloc(self.dtype, m, n)
        check(lib.prad_matmul_fwd(self._device().handle, other._device().handle, out.handle))
        if alpha != 1.0:
            check(lib.prad_scale(out.handle, out.handle, float(alpha)))
        return Tensor._from_device(out)


class TensorReverse:
    """src/PRAD/TensorReverse.cs: holds the tensors an operation consumed and computes their gradients."""

    def __init__(self, tensors):
        self.InitialTensors = list(tensors)

    def MatrixMultiplyReverse(self, upstreamGradient):
        if len(self.InitialTensors) != 2:
            raise InvalidOperationException("MatrixMultiplyReverse expects exactly two initial tensors.")
        a, b = self.InitialTensors
        if len(a.Shape) != 2 or len(b.Shape) != 2:
            raise ArgumentException("Matrix multiplication gradients are only supported for 2D tensors.")
        m, k, n = a.Shape[0], a.Shape[1], b.Shape[1]
        if k != b.Shape[0]:
            raise ArgumentException("Incompatible shapes for matrix multiplication.")
        _ensure_initialized()
        d_a, d_b = DeviceBuffer.alloc(a.dtype, m, k), DeviceBuffer.alloc(a.dtype, k, n)
        check(_lib.load().prad_matmul_bwd(upstreamGradient._device().handle, a._device().handle, b._device().handle,
                                          d_a.handle, d_b.handle, 0, 0))
        return [Tensor._from_device(d_a), Tensor._from_device(d_b)]
