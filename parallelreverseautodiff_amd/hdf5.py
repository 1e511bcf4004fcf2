"""HDF5 weight files in the reference's layout, written and read with the HDF5 C library.

Reference: src/Interprocess/HDF5Helper.cs.  The reference drives the same C library through
HDF.PInvoke, call for call as here, so the files are interchangeable:

* ``Serialize(path, matrix | [matrices])`` (:28-58, :234-269): one 1-D dataset of native doubles
  per matrix row, named ``row0, row1, ...`` in the root group, numbered through all matrices.
* ``Deserialize(path)`` (:65-114): every dataset ``row0 .. row{nlinks-1}`` as one array each.
* ``Validate(path, sizes)`` (:122-174): the file holds at least ``len(sizes)`` datasets and
  ``row{i}`` has ``sizes[i]`` elements.
* ``SerializeElements`` / ``DeserializeElements`` (:182-231, :279-325): the dictionary form that
  ModelLayer.SaveWeightsAndMomentsBinary uses: ``<path>.json`` holds the DataSet metadata
  (src/Interprocess/DataSet.cs, DataSetItem.cs: StartIndex, Rows, DeserializeKey, TypeName per
  stored object), ``<path>.hdf5`` the rows.

PRADLite's helper (lite/src/ParallelReverseAutoDiffLite/Lite/HDF5Helper.cs:39-46) hands float[]
rows to the library as native doubles, which reads past the end of every row; there is no
file layout in that to mirror.  Float matrices are written here as what was evidently meant:
their values widened to double, and narrowed again on reading.

The C library is loaded on first use: PRAD_HDF5_LIBRARY names it, otherwise the usual places are
searched.  Without it these functions raise; nothing else in the package depends on them.
"""
import ctypes
import ctypes.util
import glob
import json
import os

import numpy as np

from .exceptions import ArgumentException, InvalidOperationException
from .matrix import DeepMatrix, Matrix

hid_t = ctypes.c_int64     # HDF5 1.10 and later
herr_t = ctypes.c_int
hsize_t = ctypes.c_uint64

H5F_ACC_RDONLY = 0
H5F_ACC_TRUNC = 2
H5P_DEFAULT = 0
H5S_ALL = 0

MATRIX_TYPE_NAME = "ParallelReverseAutoDiff.RMAD.Matrix"
DEEP_MATRIX_TYPE_NAME = "ParallelReverseAutoDiff.RMAD.DeepMatrix"
DEEP_MATRIX_ARRAY_TYPE_NAME = "ParallelReverseAutoDiff.RMAD.DeepMatrix[]"


class H5G_info_t(ctypes.Structure):
    _fields_ = [("storage_type", ctypes.c_int), ("nlinks", hsize_t), ("max_corder", ctypes.c_int64),
                ("mounted", ctypes.c_uint)]


_h5 = None


def _candidates():
    named = os.environ.get("PRAD_HDF5_LIBRARY")
    if named:
        yield named
        return
    found = ctypes.util.find_library("hdf5") or ctypes.util.find_library("hdf5_serial")
    if found:
        yield found
    for pattern in ("/usr/lib/x86_64-linux-gnu/libhdf5_serial.so*", "/usr/lib/x86_64-linux-gnu/libhdf5.so*",
                    "/usr/lib64/libhdf5.so*", "/usr/local/lib/libhdf5.so*", "/opt/conda/lib/libhdf5.so*"):
        for path in sorted(glob.glob(pattern)):
            yield path


def library():
    """The HDF5 C library with argument types set; raises InvalidOperationException when there is none."""
    global _h5
    if _h5 is not None:
        return _h5
    lib, tried = None, []
    for path in _candidates():
        try:
            lib = ctypes.CDLL(path)
            break
        except OSError as e:
            tried.append("%s (%s)" % (path, e))
    if lib is None:
        raise InvalidOperationException("no HDF5 C library found; set PRAD_HDF5_LIBRARY to libhdf5.so" +
                                        ("; tried " + "; ".join(tried) if tried else ""))
    major, minor, release = ctypes.c_uint(), ctypes.c_uint(), ctypes.c_uint()
    lib.H5get_libversion(ctypes.byref(major), ctypes.byref(minor), ctypes.byref(release))
    if (major.value, minor.value) < (1, 10):
        raise InvalidOperationException("HDF5 %d.%d: 1.10 or later is needed (64-bit identifiers)" % (major.value, minor.value))
    sig = {
        "H5open": (herr_t, []),
        "H5Fcreate": (hid_t, [ctypes.c_char_p, ctypes.c_uint, hid_t, hid_t]),
        "H5Fopen": (hid_t, [ctypes.c_char_p, ctypes.c_uint, hid_t]),
        "H5Fclose": (herr_t, [hid_t]),
        "H5Screate_simple": (hid_t, [ctypes.c_int, ctypes.POINTER(hsize_t), ctypes.POINTER(hsize_t)]),
        "H5Sclose": (herr_t, [hid_t]),
        "H5Sget_simple_extent_ndims": (ctypes.c_int, [hid_t]),
        "H5Sget_simple_extent_dims": (ctypes.c_int, [hid_t, ctypes.POINTER(hsize_t), ctypes.POINTER(hsize_t)]),
        "H5Dcreate2": (hid_t, [hid_t, ctypes.c_char_p, hid_t, hid_t, hid_t, hid_t, hid_t]),
        "H5Dopen2": (hid_t, [hid_t, ctypes.c_char_p, hid_t]),
        "H5Dget_space": (hid_t, [hid_t]),
        "H5Dwrite": (herr_t, [hid_t, hid_t, hid_t, hid_t, hid_t, ctypes.c_void_p]),
        "H5Dread": (herr_t, [hid_t, hid_t, hid_t, hid_t, hid_t, ctypes.c_void_p]),
        "H5Dclose": (herr_t, [hid_t]),
        "H5Gget_info": (herr_t, [hid_t, ctypes.POINTER(H5G_info_t)]),
        "H5Eset_auto2": (herr_t, [hid_t, ctypes.c_void_p, ctypes.c_void_p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    if lib.H5open() < 0:
        raise InvalidOperationException("H5open failed")
    lib.H5Eset_auto2(0, None, None)   # errors come back as exceptions here, not as stack dumps on stderr
    lib.NATIVE_DOUBLE = hid_t.in_dll(lib, "H5T_NATIVE_DOUBLE_g").value
    _h5 = lib
    return lib


def _check(value, what):
    if value < 0:
        raise InvalidOperationException("HDF5: %s failed" % what)
    return value


class _File:
    def __init__(self, path, create):
        self.h5 = library()
        name = os.fspath(path).encode()
        if create:
            self.id = _check(self.h5.H5Fcreate(name, H5F_ACC_TRUNC, H5P_DEFAULT, H5P_DEFAULT), "H5Fcreate(%s)" % path)
        else:
            self.id = _check(self.h5.H5Fopen(name, H5F_ACC_RDONLY, H5P_DEFAULT), "H5Fopen(%s)" % path)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.h5.H5Fclose(self.id)

    def nlinks(self):
        info = H5G_info_t()
        _check(self.h5.H5Gget_info(self.id, ctypes.byref(info)), "H5Gget_info")
        return int(info.nlinks)

    def write_row(self, n, row):
        h5 = self.h5
        row = np.ascontiguousarray(row, dtype=np.float64)
        dims = (hsize_t * 1)(row.shape[0])
        space = _check(h5.H5Screate_simple(1, dims, None), "H5Screate_simple")
        try:
            dset = _check(h5.H5Dcreate2(self.id, b"row%d" % n, h5.NATIVE_DOUBLE, space, H5P_DEFAULT, H5P_DEFAULT, H5P_DEFAULT),
                          "H5Dcreate(row%d)" % n)
            try:
                if row.shape[0]:
                    _check(h5.H5Dwrite(dset, h5.NATIVE_DOUBLE, H5S_ALL, H5S_ALL, H5P_DEFAULT, row.ctypes.data), "H5Dwrite(row%d)" % n)
            finally:
                h5.H5Dclose(dset)
        finally:
            h5.H5Sclose(space)

    def row_length(self, n):
        h5 = self.h5
        dset = _check(h5.H5Dopen2(self.id, b"row%d" % n, H5P_DEFAULT), "H5Dopen(row%d)" % n)
        try:
            return self._length(dset, n)
        finally:
            h5.H5Dclose(dset)

    def _length(self, dset, n):
        h5 = self.h5
        space = _check(h5.H5Dget_space(dset), "H5Dget_space")
        try:
            if h5.H5Sget_simple_extent_ndims(space) != 1:
                raise InvalidOperationException("HDF5: row%d is not one-dimensional" % n)
            dims = (hsize_t * 1)()
            _check(h5.H5Sget_simple_extent_dims(space, dims, None), "H5Sget_simple_extent_dims")
            return int(dims[0])
        finally:
            h5.H5Sclose(space)

    def read_row(self, n):
        h5 = self.h5
        dset = _check(h5.H5Dopen2(self.id, b"row%d" % n, H5P_DEFAULT), "H5Dopen(row%d)" % n)
        try:
            out = np.empty(self._length(dset, n), dtype=np.float64)
            if out.shape[0]:
                _check(h5.H5Dread(dset, h5.NATIVE_DOUBLE, H5S_ALL, H5S_ALL, H5P_DEFAULT, out.ctypes.data), "H5Dread(row%d)" % n)
            return out
        finally:
            h5.H5Dclose(dset)


def _rows_of(matrix):
    return matrix.ToArray()


def Serialize(path, matrices):
    """HDF5Helper.Serialize(FileInfo, Matrix) and (FileInfo, List<Matrix>): src/Interprocess/HDF5Helper.cs:28-58, :234-269."""
    if isinstance(matrices, Matrix):
        matrices = [matrices]
    with _File(path, create=True) as f:
        n = 0
        for matrix in matrices:
            for row in _rows_of(matrix):
                f.write_row(n, row)
                n += 1


def Deserialize(path):
    """HDF5Helper.Deserialize(FileInfo): the rows of the file, in order (src/Interprocess/HDF5Helper.cs:65-114)."""
    with _File(path, create=False) as f:
        return [f.read_row(i) for i in range(f.nlinks())]


def Validate(path, sizes):
    """HDF5Helper.Validate (src/Interprocess/HDF5Helper.cs:122-174)."""
    sizes = list(sizes)
    with _File(path, create=False) as f:
        links = f.nlinks()
        for i, size in enumerate(sizes):
            if i >= links or f.row_length(i) != size:
                return False
        return True


def ParseObject(o):
    """(matrices, type name) of a Matrix, DeepMatrix or list of DeepMatrix (src/Interprocess/HDF5Helper.cs:332-350)."""
    if isinstance(o, Matrix):
        return [o], MATRIX_TYPE_NAME
    if isinstance(o, DeepMatrix):
        return list(o), DEEP_MATRIX_TYPE_NAME
    if isinstance(o, (list, tuple)) and len(o) > 0 and all(isinstance(d, DeepMatrix) for d in o):
        return [m for d in o for m in d], DEEP_MATRIX_ARRAY_TYPE_NAME
    raise ArgumentException("Object must be a Matrix, DeepMatrix, or DeepMatrix[].")


def SerializeElements(path, elements, gets):
    """HDF5Helper.Serialize<T>(FileInfo, IDictionary<string,T>, Func<T,object>[]) (src/Interprocess/HDF5Helper.cs:279-325):
    writes <path>.json and <path>.hdf5 and returns what Validate says of the latter."""
    matrices, items, index = [], [], 0
    for key, value in elements.items():
        for i, get in enumerate(gets):
            found, type_name = ParseObject(get(value))
            rows = sum(m.Rows for m in found)
            items.append({"StartIndex": index, "Rows": rows, "DeserializeKey": {"Item1": key, "Item2": i}, "TypeName": type_name})
            matrices.extend(found)
            index += rows
    with open(os.fspath(path) + ".json", "w") as f:
        json.dump({"Items": items}, f, indent=2)
    binary = os.fspath(path) + ".hdf5"
    Serialize(binary, matrices)
    return Validate(binary, [m.Cols for m in matrices for _ in range(m.Rows)])


def _replace(matrix, rows):
    if len(rows) != matrix.Rows or any(r.shape[0] != matrix.Cols for r in rows):
        # The reference swaps the row arrays in without looking; a stored shape that differs from the
        # element's would surface later as an index error.  Say so here instead.
        raise InvalidOperationException("stored rows do not match the %dx%d element" % (matrix.Rows, matrix.Cols))
    matrix.Replace([np.ascontiguousarray(r, dtype=matrix.dtype) for r in rows])


def _replace_deep(deep, rows):
    skip = 0
    for m in deep:
        _replace(m, rows[skip:skip + m.Rows])
        skip += m.Rows


def DeserializeElements(path, elements, gets):
    """HDF5Helper.Deserialize<T> (src/Interprocess/HDF5Helper.cs:182-231): the stored rows replace, in place, the rows
    of the objects that gets[index](elements[key]) returns."""
    with open(os.fspath(path) + ".json") as f:
        data_set = json.load(f)
    if data_set is None:
        raise InvalidOperationException("Could not deserialize metadata.")
    rows = Deserialize(os.fspath(path) + ".hdf5")
    for item in data_set["Items"]:
        key, index = item["DeserializeKey"]["Item1"], item["DeserializeKey"]["Item2"]
        mine = rows[item["StartIndex"]:item["StartIndex"] + item["Rows"]]
        target = gets[index](elements[key])
        if item["TypeName"] == MATRIX_TYPE_NAME:
            _replace(target, mine)
        elif item["TypeName"] == DEEP_MATRIX_TYPE_NAME:
            _replace_deep(target, mine)
        elif item["TypeName"] == DEEP_MATRIX_ARRAY_TYPE_NAME:
            skip = 0
            for deep in target:
                total = sum(m.Rows for m in deep)
                _replace_deep(deep, mine[skip:skip + total])
                skip += total
        else:
            raise InvalidOperationException("Unknown type name: %s" % item["TypeName"])
