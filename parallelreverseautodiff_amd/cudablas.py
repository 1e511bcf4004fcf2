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
        # set once the library has said it is initialised, cleared by Dispose: lets the operations skip one library call
        # per Forward / Backward.  (A shutdown behind this object's back is still caught: every entry point then returns
        # the not-initialised status.)
        self.known_ready = False

    @property
    def IsInitialized(self):
        self.known_ready = bool(_lib.load().prad_is_initialized())
        return self.known_ready

    def Initialize(self):
        check(_lib.load().prad_init(int(self.DeviceId)))
        self.known_ready = True

    def Dispose(self):
        self.known_ready = False
        check(_lib.load().prad_shutdown())

    def Synchronize(self):
        check(_lib.load().prad_stream_sync())


class CudaBlas:
    Instance = _CudaBlas()
