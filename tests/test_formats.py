"""Wire and file formats of Matrix / DeepMatrix / ModelLayer (host logic; no GPU):
Matrix.Serialize byte layout (src/RMAD/Matrix.cs:856-877, read back by CudaBlas.cs:355-381 and
Matrix.DeserializeToFlatArray :357-374), the Newtonsoft JSON of MatrixJsonConverter / DeepMatrixJsonConverter, and
ModelLayer.SaveWeights / SaveWeightsAndMoments / SaveWeightsAndMomentsBinary (src/RMAD/ModelLayer.cs:219-320; the
HDF5 files of src/Interprocess/HDF5Helper.cs).  The JSON reader is pinned by Matrix
objects taken from the reference's own test data (tests/golden/reference_matrix_json.json)."""
import json
import os
import struct

import numpy as np
import pytest

from parallelreverseautodiff_amd.exceptions import InvalidOperationException
from parallelreverseautodiff_amd.matrix import DeepMatrix, Matrix
from parallelreverseautodiff_amd.optim import ModelLayer

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_serialize_byte_layout(dtype):
    m = Matrix.from_numpy(np.array([[1.5, -2.0, 3.25], [4.0, 5.0, -6.5]], dtype=dtype))
    m.UniqueId = 0x01020304
    raw = m.Serialize(transpose=True)
    es = np.dtype(dtype).itemsize
    assert len(raw) == 1 + 3 * 4 + 6 * es                      # CudaBlas.cs:367: 1 + 3 * sizeof(int) + rows * cols * sizeof(T)
    assert raw[0] == 1
    assert raw[1:5] == bytes([4, 3, 2, 1])                     # little-endian int32 UniqueId
    assert struct.unpack_from("<ii", raw, 5) == (2, 3)
    fmt = "<6d" if dtype == np.float64 else "<6f"
    assert struct.unpack_from(fmt, raw, 13) == (1.5, -2.0, 3.25, 4.0, 5.0, -6.5)   # row-major payload
    assert Matrix(2, 3, dtype).Serialize()[0] == 0
    flat = Matrix.DeserializeToFlatArray(raw, dtype)
    assert flat.dtype == dtype and np.array_equal(flat, [1.5, -2.0, 3.25, 4.0, 5.0, -6.5])
    flag, back = Matrix.Deserialize(raw, dtype)
    assert flag is True and back.UniqueId == 0x01020304 and np.array_equal(back.to_numpy(), m.to_numpy())


def test_reads_matrices_written_by_the_reference():
    with open(os.path.join(HERE, "golden", "reference_matrix_json.json")) as f:
        fixture = json.load(f)
    first = Matrix.from_json_object(fixture["matrices"][0])
    assert first.UniqueId == 3865291 and (first.Rows, first.Cols) == (16, 1)
    assert [first[i, 0] for i in range(4)] == [112.0, 88.0, 97.0, 100.0]
    for obj in fixture["matrices"]:
        m = Matrix.from_json_object(obj)
        again = m.to_json_object()
        assert again["UniqueId"] == obj["UniqueId"] and again["MatrixValues"] == obj["MatrixValues"]
        assert again["Shape"] == [m.Rows, m.Cols] and again["NumDimensions"] == 2   # written by current versions


def test_deep_matrix_json_round_trip():
    d = DeepMatrix.from_numpy(np.arange(24, dtype=np.float64).reshape(2, 3, 4))
    obj = json.loads(json.dumps(d.to_json_object()))
    assert set(obj) == {"UniqueId", "MatrixArrayValues"} and len(obj["MatrixArrayValues"]) == 2
    back = DeepMatrix.from_json_object(obj)
    assert back.UniqueId == d.UniqueId and np.array_equal(back.to_numpy(), d.to_numpy())
    assert [m.UniqueId for m in back] == [m.UniqueId for m in d]


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_model_layer_files_round_trip(tmp_path, dtype):
    rng = np.random.default_rng(5)
    mk = lambda *shape: rng.standard_normal(shape).astype(dtype)
    src = ModelLayer()
    src.AddModelElementGroup("W", Matrix.from_numpy(mk(5, 7)), None, Matrix.from_numpy(mk(5, 7)), Matrix.from_numpy(mk(5, 7)))
    src.AddModelElementGroup("K", DeepMatrix.from_numpy(mk(3, 2, 4)), None, DeepMatrix.from_numpy(mk(3, 2, 4)), DeepMatrix.from_numpy(mk(3, 2, 4)))
    path = str(tmp_path / "layer.json")
    src.SaveWeightsAndMoments(path)
    with open(path) as f:
        text = json.load(f)
    assert list(text) == ["Item1", "Item2", "Item3"] and list(text["Item1"]) == ["W", "K"]    # a ValueTuple of three dictionaries
    assert set(text["Item1"]["W"]) == {"UniqueId", "MatrixValues", "Shape", "NumDimensions"}
    dst = ModelLayer()
    dst.AddModelElementGroup("W", Matrix(5, 7, dtype))
    dst.AddModelElementGroup("K", DeepMatrix(3, 2, 4, dtype))
    dst.AddModelElementGroup("extra", Matrix(1, 1, dtype))      # not in the file: left alone
    dst.LoadWeightsAndMoments(path)
    for ident in ("W", "K"):
        for element in ("Weight", "FirstMoment", "SecondMoment"):
            got, want = dst[ident, element], src[ident, element]
            assert got.dtype == dtype and np.array_equal(got.to_numpy(), want.to_numpy())   # float values round-trip exactly
    assert np.array_equal(dst["extra", "Weight"].to_numpy(), np.zeros((1, 1), dtype))
    wpath = str(tmp_path / "weights.json")
    src.SaveWeights(wpath)
    with open(wpath) as f:
        assert list(json.load(f)) == ["W", "K"]
    only = ModelLayer().AddModelElementGroup("W", Matrix(5, 7, dtype))
    only.LoadWeights(wpath)
    assert np.array_equal(only["W", "Weight"].to_numpy(), src["W", "Weight"].to_numpy())


# ---- HDF5 files (src/Interprocess/HDF5Helper.cs), through the HDF5 C library that the reference also calls ----
def _hdf5():
    from parallelreverseautodiff_amd import hdf5
    from parallelreverseautodiff_amd.exceptions import InvalidOperationException
    try:
        hdf5.library()
    except InvalidOperationException as e:
        pytest.skip(str(e))
    return hdf5


def test_hdf5_rows_are_native_double_datasets(tmp_path):
    hdf5 = _hdf5()
    rng = np.random.default_rng(11)
    a, b = rng.standard_normal((3, 5)), rng.standard_normal((2, 7))
    path = str(tmp_path / "m.hdf5")
    hdf5.Serialize(path, [Matrix.from_numpy(a), Matrix.from_numpy(b)])
    raw = open(path, "rb").read()
    assert raw[:8] == b"\x89HDF\r\n\x1a\n"
    # Independent of the reader: every row lies in the file as contiguous little-endian doubles, and the
    # datasets are named row0.. through both matrices.
    for row in list(a) + list(b):
        assert row.astype("<f8").tobytes() in raw
    for n in range(5):
        assert b"row%d\x00" % n in raw
    assert b"row5\x00" not in raw
    rows = hdf5.Deserialize(path)
    assert [r.shape[0] for r in rows] == [5, 5, 5, 7, 7]
    assert np.array_equal(np.stack(rows[:3]), a) and np.array_equal(np.stack(rows[3:]), b)
    assert hdf5.Validate(path, [5, 5, 5, 7, 7]) and hdf5.Validate(path, [5, 5])     # fewer sizes than rows is valid
    assert not hdf5.Validate(path, [5, 5, 5, 7, 8]) and not hdf5.Validate(path, [5, 5, 5, 7, 7, 7])
    hdf5.Serialize(path, Matrix.from_numpy(a))                                        # truncates
    assert len(hdf5.Deserialize(path)) == 3


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_model_layer_binary_files_round_trip(tmp_path, dtype):
    hdf5 = _hdf5()
    rng = np.random.default_rng(6)
    mk = lambda *shape: rng.standard_normal(shape).astype(dtype)
    src = ModelLayer()
    src.AddModelElementGroup("W", Matrix.from_numpy(mk(5, 7)), None, Matrix.from_numpy(mk(5, 7)), Matrix.from_numpy(mk(5, 7)))
    src.AddModelElementGroup("K", DeepMatrix.from_numpy(mk(3, 2, 4)), None, DeepMatrix.from_numpy(mk(3, 2, 4)), DeepMatrix.from_numpy(mk(3, 2, 4)))
    path = str(tmp_path / "layer")
    src.SaveWeightsAndMomentsBinary(path)
    with open(path + ".json") as f:
        meta = json.load(f)
    # DataSet / DataSetItem as Newtonsoft writes them; rows are numbered through weight, first moment,
    # second moment of each identifier in turn.
    assert list(meta) == ["Items"] and len(meta["Items"]) == 6
    assert [list(i) for i in meta["Items"]] == [["StartIndex", "Rows", "DeserializeKey", "TypeName"]] * 6
    assert [(i["DeserializeKey"]["Item1"], i["DeserializeKey"]["Item2"]) for i in meta["Items"]] == \
        [("W", 0), ("W", 1), ("W", 2), ("K", 0), ("K", 1), ("K", 2)]
    assert [i["StartIndex"] for i in meta["Items"]] == [0, 5, 10, 15, 21, 27] and [i["Rows"] for i in meta["Items"]] == [5, 5, 5, 6, 6, 6]
    assert [i["TypeName"] for i in meta["Items"]] == ["ParallelReverseAutoDiff.RMAD.Matrix"] * 3 + ["ParallelReverseAutoDiff.RMAD.DeepMatrix"] * 3
    rows = hdf5.Deserialize(path + ".hdf5")
    assert len(rows) == 33 and np.array_equal(np.stack(rows[5:10]), src["W", "FirstMoment"].to_numpy().astype(np.float64))
    dst = ModelLayer()
    dst.AddModelElementGroup("W", Matrix(5, 7, dtype))
    dst.AddModelElementGroup("K", DeepMatrix(3, 2, 4, dtype))
    kept = dst["K", "Weight"]
    dst.LoadWeightsAndMomentsBinary(path)
    assert dst["K", "Weight"] is kept                      # rows are replaced inside the existing objects
    for ident in ("W", "K"):
        for element in ("Weight", "FirstMoment", "SecondMoment"):
            got, want = dst[ident, element], src[ident, element]
            assert got.dtype == dtype and np.array_equal(got.to_numpy(), want.to_numpy())
    wrong = ModelLayer().AddModelElementGroup("W", Matrix(5, 8, dtype)).AddModelElementGroup("K", DeepMatrix(3, 2, 4, dtype))
    with pytest.raises(InvalidOperationException):
        wrong.LoadWeightsAndMomentsBinary(path)
