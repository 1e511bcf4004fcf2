"""CudaBlas.Instance facade (src/RMAD/CudaBlas.cs:71-155) mapped onto prad_init / prad_shutdown.

Every example and test of the reference brackets GPU work with
``CudaBlas.Instance.DeviceId = 0; CudaBlas.Instance.Initialize(); ...; CudaBlas.Instance.Dispose()``
(examples/feedforward/ParallelReverseAutoDiff.FeedForwardExample/Program.cs:17-25).  The name is kept so that
code reads the same; what it starts is the HIP library, not cuBLAS.
"""
from . import _lib
from .exceptions import check


class _CudaBlas:
    def __init__(self):
        self.DeviceId = 0

    @property
    def IsInitialized(self):
        return bool(_lib.load().prad_is_initialized())

    def Initialize(self):
        check(_lib.load().prad_init(int(self.DeviceId)))

    def Dispose(self):
        check(_lib.load().prad_shutdown())

    def Synchronize(self):
        check(_lib.load().prad_stream_sync())


class CudaBlas:
    Instance = _CudaBlas()
