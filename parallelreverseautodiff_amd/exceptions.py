"""Exception types the reference's operations raise, and the status-code mapping of the C ABI.

The reference throws managed exceptions (src/RMAD/MatrixMultiplyOperation.cs:59-62,
src/RMAD/GpuMatrixMultiplyOperation.cs:115-118, :177-180, :244-247, src/RMAD/CudaBlas.cs:251-256);
the C ABI returns negative status codes and this module turns them back into the same types
with the same messages.
"""
from . import _lib


class InvalidOperationException(RuntimeError):
    pass


class ArgumentException(ValueError):
    pass


class CudaNotInitializedException(RuntimeError):
    """src/Exceptions/CudaNotInitializedException.cs"""

    def __init__(self, message="CudaBlas is not initialized."):
        super().__init__(message)


_BY_CODE = {
    _lib.PRAD_ERR_NOT_INITIALIZED: CudaNotInitializedException,
    _lib.PRAD_ERR_SHAPE: InvalidOperationException,
    _lib.PRAD_ERR_ALLOC: MemoryError,
    _lib.PRAD_ERR_LAUNCH: InvalidOperationException,
    _lib.PRAD_ERR_BAD_HANDLE: ArgumentException,
    _lib.PRAD_ERR_ARG: ArgumentException,
    _lib.PRAD_ERR_NOT_RECTANGULAR: InvalidOperationException,
    _lib.PRAD_ERR_DTYPE: ArgumentException,
    _lib.PRAD_ERR_RECORDING: InvalidOperationException,
}


def check(status):
    """Raises the exception that corresponds to a non-zero C ABI status."""
    if status == _lib.PRAD_OK:
        return
    message = _lib.load().prad_last_error().decode("utf-8", "replace")
    if status == _lib.PRAD_ERR_NOT_INITIALIZED:
        raise CudaNotInitializedException()
    raise _BY_CODE.get(status, RuntimeError)(message)
