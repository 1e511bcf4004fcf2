"""Initialize / Dispose life cycle of the library (CudaBlas.Instance.Initialize / Dispose in the reference,
src/RMAD/CudaBlas.cs:71-155), in a process of its own so that disposing does not pull the device from under the
other tests' buffers."""
import os
import subprocess
import sys
import textwrap

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SCRIPT = textwrap.dedent("""
    import ctypes, sys
    import numpy as np
    sys.path.insert(0, %r)
    from parallelreverseautodiff_amd import _lib
    from parallelreverseautodiff_amd.cudablas import CudaBlas
    from parallelreverseautodiff_amd.exceptions import ArgumentException, CudaNotInitializedException, check
    from parallelreverseautodiff_amd.matrix import Matrix
    from parallelreverseautodiff_amd.operations import GpuMatrixMultiplyOperation
    lib = _lib.load()
    blas = CudaBlas.Instance
    assert not blas.IsInitialized
    a, b = Matrix.from_numpy(np.arange(6.0).reshape(2, 3)), Matrix.from_numpy(np.ones((3, 2)))
    try:
        GpuMatrixMultiplyOperation.Instantiate(None).Forward(a, b)
        raise SystemExit("no exception before Initialize")
    except CudaNotInitializedException:
        pass
    assert lib.prad_init(99) == _lib.PRAD_ERR_ARG                      # no such device
    blas.DeviceId = 0
    blas.Initialize()
    blas.Initialize()                                                  # idempotent on the same device
    assert blas.IsInitialized and lib.prad_device_id() == 0
    assert lib.prad_init(1) == _lib.PRAD_ERR_ARG                       # already initialized on device 0
    c = GpuMatrixMultiplyOperation.Instantiate(None).Forward(a, b).to_numpy()
    assert np.array_equal(c, np.array([[3.0, 3.0], [12.0, 12.0]]))
    blas.Dispose()
    assert not blas.IsInitialized
    h = ctypes.c_void_p()
    assert lib.prad_buf_alloc(_lib.PRAD_F64, 2, 2, ctypes.byref(h)) == _lib.PRAD_ERR_NOT_INITIALIZED
    assert lib.prad_stream_sync() == _lib.PRAD_ERR_NOT_INITIALIZED
    blas.Dispose()                                                     # disposing twice is harmless
    blas.Initialize()                                                  # and the library comes back
    a2, b2 = Matrix.from_numpy(np.arange(6.0).reshape(2, 3)), Matrix.from_numpy(np.ones((3, 2)))
    c2 = GpuMatrixMultiplyOperation.Instantiate(None).Forward(a2, b2).to_numpy()
    assert np.array_equal(c2, c)
    blas.Dispose()
    print("lifecycle ok")
""") % ROOT


def test_initialize_dispose_cycle():
    proc = subprocess.run([sys.executable, "-c", SCRIPT], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=170)
    assert proc.returncode == 0 and "lifecycle ok" in proc.stdout, proc.stdout[-3000:]
