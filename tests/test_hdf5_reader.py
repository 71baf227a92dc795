"""The facade's read_hdf5 (source/util.cu:100-131 without libhdf5) on the data files the reference
itself holds: shapes, types and values against what those files are known to contain."""
import ctypes as C
import hashlib
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
DATA = os.path.join(HERE, "golden", "hdf5")


@pytest.fixture(scope="module")
def reader():
    if not os.environ.get("CNHIP_NO_TORCH"):
        import torch  # noqa: F401  (the facade links the HIP runtime; load torch's copy first)
    # CN_FACADE_LIB: another build of the facade (the host-sanitizer build)
    lib = C.CDLL(os.environ.get("CN_FACADE_LIB") or os.path.join(os.path.dirname(HERE), "clusternet_amd", "libclusternet.so"))
    fn = lib.cn_facade_read_hdf5
    fn.argtypes = [C.c_char_p, C.c_char_p, C.POINTER(C.c_longlong), C.POINTER(C.c_longlong),
                   C.POINTER(C.POINTER(C.c_float)), C.POINTER(C.c_char_p)]
    libc = C.CDLL(None)
    libc.free.argtypes = [C.c_void_p]

    def read(name, tag=None):
        rows, cols, data, err = C.c_longlong(), C.c_longlong(), C.POINTER(C.c_float)(), C.c_char_p()
        path = name if os.path.isabs(name) else os.path.join(DATA, name)
        rc = fn(path.encode(), None if tag is None else tag.encode(), C.byref(rows), C.byref(cols), C.byref(data),
                C.byref(err))
        if rc != 0:
            raise RuntimeError(err.value.decode())
        out = np.ctypeslib.as_array(data, shape=(rows.value, cols.value)).copy() if rows.value * cols.value else \
            np.empty((rows.value, cols.value), np.float32)
        libc.free(data)
        return out
    return read


def test_float64_arange_is_converted_like_h5dread(reader):
    a = reader("numpy_arange_as_h5py.hdf5")          # numpy.arange written by h5py as float64, 10 x 50
    assert a.shape == (10, 50) and a.dtype == np.float32
    assert np.array_equal(a, np.arange(500, dtype=np.float32).reshape(10, 50))
    assert np.array_equal(reader("numpy_arange_as_h5py.hdf5", "/Default"), a)
    assert np.array_equal(reader("numpy_arange_as_h5py.hdf5", "Default"), a)


def test_codec_table_file_equals_the_embedded_table(reader):
    t = reader("8bit_floats.hdf5")
    assert t.shape == (126, 1)
    want = np.fromfile(os.path.join(HERE, "golden", "8bit_floats_table.bin"), dtype=np.float32)
    assert np.array_equal(t.reshape(-1).view(np.uint32), want.view(np.uint32))
    assert hashlib.sha256(t.tobytes()).hexdigest() == hashlib.sha256(want.tobytes()).hexdigest()


def test_mnist_mini(reader):
    X, y = reader("mnist_mini_X.hdf5"), reader("mnist_mini_y.hdf5")
    assert X.shape == (500, 784) and y.shape == (500, 1)
    assert X.min() == 0.0 and 0.99 <= X.max() <= 1.0         # pixel intensities scaled to [0, 1]
    assert set(np.unique(y)) <= set(range(10)) and len(np.unique(y)) == 10
    raw = np.fromfile(os.path.join(DATA, "mnist_mini_X.hdf5"), dtype=np.float32, offset=2144, count=500 * 784)
    assert np.array_equal(X.reshape(-1).view(np.uint32), raw.view(np.uint32))


def test_named_integer_datasets(reader):
    f = "scipy_sparse_arange_as_h5py.hdf5"                    # CSR pieces of a sparse arange
    shape = reader(f, "shape")
    assert shape.shape == (2, 1) and shape.dtype == np.float32
    rows, cols = int(shape[0, 0]), int(shape[1, 0])
    indptr, indices, data = reader(f, "indptr"), reader(f, "indices"), reader(f, "data")
    assert indptr.shape == (rows + 1, 1) and indptr[0, 0] == 0 and indptr[-1, 0] == indices.shape[0] == data.shape[0]
    assert np.all(np.diff(indptr[:, 0]) >= 0) and indices.max() < cols and indices.min() >= 0


def test_refusals_are_messages_not_crashes(reader, tmp_path):
    with pytest.raises(RuntimeError, match="no dataset of that name"):
        reader("numpy_arange_as_h5py.hdf5", "Missing")
    with pytest.raises(RuntimeError, match="cannot open"):
        reader(str(tmp_path / "nope.hdf5"))
    junk = tmp_path / "junk.hdf5"
    junk.write_bytes(b"not an hdf5 file" * 10)
    with pytest.raises(RuntimeError, match="not an HDF5 file"):
        reader(str(junk))
    whole = open(os.path.join(DATA, "mnist_mini_y.hdf5"), "rb").read()
    cut = tmp_path / "cut.hdf5"
    cut.write_bytes(whole[:3000])                              # payload truncated
    with pytest.raises(RuntimeError, match="outside the file"):
        reader(str(cut))
