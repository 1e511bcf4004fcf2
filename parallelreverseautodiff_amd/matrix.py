"""Matrix / DeepMatrix: the reference's jagged host containers with a device-resident twin.

Reference: src/RMAD/Matrix.cs:25-55 (``double[][] matrix``, one array per row, ``UniqueId``),
src/RMAD/DeepMatrix.cs:22 (an array of Matrix).  PRADLite uses ``float[][]``
(lite/src/ParallelReverseAutoDiffLite/Lite/Matrix.cs).

Residency protocol.  A Matrix may hold its values on the host (a list of per-row arrays, as in
the reference), on the device (a dense row-major buffer of libprad_hip), or both.  Operations
read and write the device copy; the jagged host copy is marshalled once per direction and only
when needed:
  * ``device()`` uploads the rows if the host copy is newer (or the only one);
  * any host access (``m[i]``, iteration, ``ToArray()``) first downloads if the device copy is
    newer, and - because the reference hands out live row arrays that callers mutate in place
    (OperationBase.AccumulateGradient, AdamOptimizer, GradientClearer) - marks the device copy
    stale.  ``to_numpy()`` reads without invalidating.
"""
import ctypes
import itertools
import struct
import threading

import numpy as np

from . import _lib
from .exceptions import ArgumentException, InvalidOperationException, check

_id_lock = threading.Lock()
_id_counter = itertools.count(1)


def _next_id():
    # PseudoUniqueIDGenerator (src/Interprocess/PseudoUniqueIDGenerator.cs:28-39): a process-wide counter.
    with _id_lock:
        return next(_id_counter)


def _dtype_code(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float64:
        return _lib.PRAD_F64
    if dtype == np.float32:
        return _lib.PRAD_F32
    raise ArgumentException("element type must be float64 (PRAD) or float32 (PRADLite)")


class DeviceBuffer:
    """Owning (or borrowing) wrapper of a prad_buf_t handle."""

    def __init__(self, handle, dtype, depth, rows, cols, parent=None):
        self.handle = handle
        self.dtype = np.dtype(dtype)
        self.depth, self.rows, self.cols = depth, rows, cols
        self._parent = parent  # keeps the owner of borrowed memory alive

    @classmethod
    def alloc(cls, dtype, rows, cols, depth=1):
        """A zero-filled buffer, like new Matrix(rows, cols)."""
        lib = _lib.load()
        h = ctypes.c_void_p()
        check(lib.prad_buf_alloc_deep(_dtype_code(dtype), depth, rows, cols, ctypes.byref(h)))
        return cls(h, dtype, depth, rows, cols)

    @classmethod
    def alloc_output(cls, dtype, rows, cols, depth=1):
        """A buffer whose contents are undefined until the next kernel overwrites all of it (no fill launch)."""
        lib = _lib.load()
        h = ctypes.c_void_p()
        check(lib.prad_buf_alloc_output(_dtype_code(dtype), depth, rows, cols, ctypes.byref(h)))
        return cls(h, dtype, depth, rows, cols)

    def slice(self, d):
        """A borrowed 2-D view of slice d of a deep buffer."""
        lib = _lib.load()
        base = lib.prad_buf_device_ptr(self.handle)
        off = d * self.rows * self.cols * self.dtype.itemsize
        h = ctypes.c_void_p()
        check(lib.prad_buf_wrap(_dtype_code(self.dtype), self.rows, self.cols, ctypes.c_void_p(base + off), ctypes.byref(h)))
        return DeviceBuffer(h, self.dtype, 1, self.rows, self.cols, parent=self)

    def view_rows(self, row0, rows):
        """A borrowed view of rows [row0, row0 + rows) of a 2-D buffer."""
        h = ctypes.c_void_p()
        check(_lib.load().prad_buf_view_rows(self.handle, row0, rows, ctypes.byref(h)))
        return DeviceBuffer(h, self.dtype, 1, rows, self.cols, parent=self)

    @property
    def ptr(self):
        return _lib.load().prad_buf_device_ptr(self.handle)

    def upload(self, array):
        array = np.ascontiguousarray(array, dtype=self.dtype).reshape(self.depth * self.rows, self.cols)
        check(_lib.load().prad_buf_upload(self.handle, array.ctypes.data, self.cols))

    def upload_rows(self, rows):
        n = len(rows)
        ptrs = (ctypes.c_void_p * n)(*[r.ctypes.data for r in rows])
        lens = (ctypes.c_int64 * n)(*[r.shape[0] for r in rows])
        check(_lib.load().prad_buf_upload_rows(self.handle, ptrs, lens))

    def download(self):
        out = np.empty((self.depth * self.rows, self.cols), dtype=self.dtype)
        check(_lib.load().prad_buf_download(self.handle, out.ctypes.data, self.cols))
        return out.reshape((self.depth, self.rows, self.cols)) if self.depth > 1 else out

    def download_rows(self, rows):
        n = len(rows)
        ptrs = (ctypes.c_void_p * n)(*[r.ctypes.data for r in rows])
        check(_lib.load().prad_buf_download_rows(self.handle, ptrs))

    def zero(self):
        check(_lib.load().prad_buf_zero(self.handle))

    def __del__(self):
        try:
            lib = _lib.load()
            if self.handle is not None and lib.prad_is_initialized():
                lib.prad_buf_free(self.handle)
        except Exception:
            pass
        self.handle = None


class Matrix:
    """Jagged rows x cols matrix of float64 (PRAD) or float32 (PRADLite)."""

    def __init__(self, rows, cols=None, dtype=np.float64):
        self.UniqueId = _next_id()
        self._dev = None
        self._dev_valid = False
        if cols is None:
            # Matrix(double[][]): adopts the given row arrays (src/RMAD/Matrix.cs:60-63).
            given = list(rows)
            if len(given) == 0:
                raise ArgumentException("matrix needs at least one row")
            first = np.asarray(given[0])
            self.dtype = np.dtype(first.dtype if first.dtype in (np.float32, np.float64) else dtype)
            self._rows = [self._adopt_row(r) for r in given]
            self._nrows, self._ncols = len(self._rows), self._rows[0].shape[0]
        else:
            if rows <= 0 or cols <= 0:
                raise ArgumentException("matrix dimensions must be positive")
            self.dtype = np.dtype(dtype)
            _dtype_code(self.dtype)
            self._nrows, self._ncols = int(rows), int(cols)
            self._rows = [np.zeros(self._ncols, dtype=self.dtype) for _ in range(self._nrows)]  # one array per row
        self._host_valid = True

    def _adopt_row(self, r):
        """A row array as the device copies read it: one-dimensional, contiguous, of this matrix's element type.  An
        array that already is (the usual case) is adopted as it is and stays live, like a row of the reference's
        double[][]; a strided view or an array of another type is copied."""
        if isinstance(r, np.ndarray) and r.dtype == self.dtype and r.ndim == 1 and r.flags["C_CONTIGUOUS"]:
            return r
        return np.ascontiguousarray(np.asarray(r, dtype=self.dtype).reshape(-1))

    # ---- construction helpers -------------------------------------------------------------
    @classmethod
    def from_numpy(cls, array):
        array = np.asarray(array)
        if array.ndim != 2:
            raise ArgumentException("expected a 2-D array")
        dtype = array.dtype if array.dtype in (np.float32, np.float64) else np.float64
        return cls([np.array(array[i], dtype=dtype) for i in range(array.shape[0])])

    @classmethod
    def _from_device(cls, dev):
        m = cls.__new__(cls)
        m.UniqueId = _next_id()
        m.dtype = dev.dtype
        m._nrows, m._ncols = dev.rows, dev.cols
        m._rows = None
        m._host_valid = False
        m._dev = dev
        m._dev_valid = True
        return m

    # ---- reference surface ----------------------------------------------------------------
    @property
    def Rows(self):
        return self._nrows

    @property
    def Cols(self):
        return self._ncols

    @property
    def Length(self):
        return self._nrows

    def __len__(self):
        return self._nrows

    def _host(self, will_write=True):
        if not self._host_valid:
            if self._rows is None:
                self._rows = [np.empty(self._ncols, dtype=self.dtype) for _ in range(self._nrows)]
            self._dev.download_rows(self._rows)
            self._host_valid = True
        if will_write:
            self._dev_valid = False
        return self._rows

    def __getitem__(self, index):
        if isinstance(index, tuple):
            i, j = index
            return self._host(will_write=False)[i][j]
        return self._host()[index]

    def __setitem__(self, index, value):
        rows = self._host()
        if isinstance(index, tuple):
            i, j = index
            rows[i][j] = value
        else:
            rows[index] = self._adopt_row(value)  # row replacement, as GradientClearer does

    def __iter__(self):
        return iter(self._host())

    def ToArray(self):
        return self._host()

    def Replace(self, rows):
        self._rows = [self._adopt_row(r) for r in rows]
        self._nrows, self._ncols = len(self._rows), self._rows[0].shape[0]
        self._host_valid, self._dev_valid = True, False
        if self._dev is not None and (self._dev.rows != self._nrows or self._dev.cols != self._ncols):
            self._dev = None

    # ---- device side ------------------------------------------------------------------------
    def device(self):
        """Device buffer holding the current values (uploads the jagged rows when needed).  Row arrays handed out
        before this call stay live on the host only: fetch them again (m[i], ToArray()) before writing, which marks
        the device copy stale."""
        if self._dev is None:
            self._dev = DeviceBuffer.alloc(self.dtype, self._nrows, self._ncols)
            self._dev_valid = False
        if not self._dev_valid:
            rows = self._rows
            if len(rows) != self._nrows or any(r.shape[0] != self._ncols for r in rows):
                raise InvalidOperationException("The given jagged array is not rectangular.")
            self._dev.upload_rows(rows)
            self._dev_valid = True
        return self._dev

    def _device_written(self):
        self._dev_valid, self._host_valid = True, False

    def to_numpy(self):
        """Dense copy of the current values; does not invalidate the device copy."""
        if self._host_valid:
            return np.stack(self._rows)
        return self._dev.download()

    # ---- wire and file formats ------------------------------------------------------------------
    def Serialize(self, transpose=False):
        """The byte layout of Matrix.Serialize (src/RMAD/Matrix.cs:856-877; float elements in PRADLite): one byte
        transpose flag, int32 UniqueId, int32 Rows, int32 Cols (little endian, as BitConverter writes on x64), then
        the values row-major.  The flag is carried, not applied."""
        head = struct.pack("<Biii", 1 if transpose else 0, int(self.UniqueId), self._nrows, self._ncols)
        return head + np.ascontiguousarray(self.to_numpy(), dtype=self.dtype.newbyteorder("<")).tobytes()

    @staticmethod
    def DeserializeToFlatArray(buffer, dtype=np.float64):
        """Matrix.DeserializeToFlatArray (src/RMAD/Matrix.cs:357-374): the values of a serialized matrix as one flat array."""
        _, _, rows, cols = struct.unpack_from("<Biii", buffer, 0)
        return np.frombuffer(buffer, dtype=np.dtype(dtype).newbyteorder("<"), count=rows * cols, offset=13).astype(dtype)

    @classmethod
    def Deserialize(cls, buffer, dtype=np.float64):
        """(transpose flag, Matrix) from the byte layout of Serialize; the UniqueId travels with the matrix."""
        flag, uid, rows, cols = struct.unpack_from("<Biii", buffer, 0)
        m = cls.from_numpy(cls.DeserializeToFlatArray(buffer, dtype).reshape(rows, cols))
        m.UniqueId = uid
        return bool(flag), m

    def to_json_object(self):
        """What MatrixJsonConverter.WriteJson emits (src/RMAD/MatrixJsonConverter.cs:34-47)."""
        return {"UniqueId": int(self.UniqueId), "MatrixValues": [[float(v) for v in row] for row in self.to_numpy()],
                "Shape": [self._nrows, self._ncols], "NumDimensions": 2}

    @classmethod
    def from_json_object(cls, obj, dtype=np.float64):
        """MatrixJsonConverter.ReadJson (src/RMAD/MatrixJsonConverter.cs:57-72); Shape and NumDimensions are optional,
        as in files written by older versions."""
        values = obj["MatrixValues"]
        m = cls([np.array(row, dtype=dtype) for row in values])
        m.UniqueId = int(obj["UniqueId"])
        return m


class DeepMatrix:
    """Array of Matrix (src/RMAD/DeepMatrix.cs:22) whose device twin is one contiguous deep buffer."""

    def __init__(self, depth, rows=None, cols=None, dtype=np.float64):
        self.UniqueId = _next_id()
        self._dev = None
        if rows is None:
            self._mats = list(depth)  # DeepMatrix(Matrix[])
            if len(self._mats) == 0:
                raise ArgumentException("deep matrix needs at least one slice")
        else:
            self._mats = [Matrix(rows, cols, dtype) for _ in range(depth)]
        self.dtype = self._mats[0].dtype

    @classmethod
    def from_numpy(cls, array):
        array = np.asarray(array)
        if array.ndim != 3:
            raise ArgumentException("expected a 3-D array")
        return cls([Matrix.from_numpy(array[d]) for d in range(array.shape[0])])

    @classmethod
    def _from_device(cls, dev):
        dm = cls.__new__(cls)
        dm.UniqueId = _next_id()
        dm.dtype = dev.dtype
        dm._dev = dev
        dm._mats = [Matrix._from_device(dev.slice(d)) for d in range(dev.depth)]
        return dm

    @property
    def Depth(self):
        return len(self._mats)

    @property
    def Rows(self):
        return self._mats[0].Rows

    @property
    def Cols(self):
        return self._mats[0].Cols

    def __len__(self):
        return len(self._mats)

    def __getitem__(self, d):
        return self._mats[d]

    def __setitem__(self, d, m):
        self._mats[d] = m
        self._dev = None

    def __iter__(self):
        return iter(self._mats)

    def device(self):
        """Contiguous deep buffer with the current values of every slice."""
        fresh = self._dev is not None and all(
            m._dev is not None and m._dev._parent is self._dev and m._dev_valid for m in self._mats)
        if fresh:
            return self._dev
        dev = DeviceBuffer.alloc(self.dtype, self.Rows, self.Cols, depth=self.Depth)
        dev.upload(np.stack([m.to_numpy() for m in self._mats]))
        self._dev = dev
        for d, m in enumerate(self._mats):
            m._dev = dev.slice(d)
            m._dev_valid = True
        return dev

    def to_numpy(self):
        return np.stack([m.to_numpy() for m in self._mats])

    def to_json_object(self):
        """DeepMatrixJsonConverter.WriteJson (src/RMAD/DeepMatrixJsonConverter.cs:33-42)."""
        return {"UniqueId": int(self.UniqueId), "MatrixArrayValues": [m.to_json_object() for m in self._mats]}

    @classmethod
    def from_json_object(cls, obj, dtype=np.float64):
        d = cls([Matrix.from_json_object(o, dtype) for o in obj["MatrixArrayValues"]])
        d.UniqueId = int(obj["UniqueId"])
        return d
