"""Minimal read-only hdf5 access for the tests (h5py is not installed): ctypes on the HDF5 C
library that the host executables link."""

import ctypes as C
import glob
import os

import numpy as np

_cands = sorted(glob.glob("/opt/conda/lib/libhdf5.so.[0-9]*")) + ["/opt/conda/lib/libhdf5.so"]
_path = next((p for p in _cands if os.path.exists(p)), None)
available = _path is not None
if available:
    _h = C.CDLL(_path)
    _h.H5open()
    hid = C.c_int64
    for name, res, args in [
        ("H5Fopen", hid, [C.c_char_p, C.c_uint, hid]),
        ("H5Fclose", C.c_int, [hid]),
        ("H5Dopen2", hid, [hid, C.c_char_p, hid]),
        ("H5Dclose", C.c_int, [hid]),
        ("H5Dget_space", hid, [hid]),
        ("H5Dget_type", hid, [hid]),
        ("H5Dread", C.c_int, [hid, hid, hid, hid, hid, C.c_void_p]),
        ("H5Sget_simple_extent_ndims", C.c_int, [hid]),
        ("H5Sget_simple_extent_dims", C.c_int, [hid, C.c_void_p, C.c_void_p]),
        ("H5Sclose", C.c_int, [hid]),
        ("H5Tget_class", C.c_int, [hid]),
        ("H5Tget_size", C.c_size_t, [hid]),
        ("H5Tclose", C.c_int, [hid]),
        ("H5Oopen", hid, [hid, C.c_char_p, hid]),
        ("H5Oclose", C.c_int, [hid]),
        ("H5Aopen_name", hid, [hid, C.c_char_p]),
        ("H5Aget_space", hid, [hid]),
        ("H5Aget_type", hid, [hid]),
        ("H5Aread", C.c_int, [hid, hid, C.c_void_p]),
        ("H5Aclose", C.c_int, [hid]),
        ("H5Lexists", C.c_int, [hid, C.c_char_p, hid]),
    ]:
        f = getattr(_h, name)
        f.restype, f.argtypes = res, args
    _native = {
        (0, 4): ("H5T_NATIVE_INT32_g", np.int32),
        (0, 8): ("H5T_NATIVE_INT64_g", np.int64),
        (1, 4): ("H5T_NATIVE_FLOAT_g", np.float32),
        (1, 8): ("H5T_NATIVE_DOUBLE_g", np.float64),
    }

    def _mem(tid):
        sym, dt = _native[(_h.H5Tget_class(tid), _h.H5Tget_size(tid))]
        return hid.in_dll(_h, sym).value, dt

    def _dims(sid):
        nd = _h.H5Sget_simple_extent_ndims(sid)
        dims = (C.c_uint64 * max(nd, 1))()
        if nd > 0:
            _h.H5Sget_simple_extent_dims(sid, dims, None)
        return tuple(int(dims[i]) for i in range(nd))

    def read(path, name):
        """Dataset -> numpy array with the file's own dtype and shape."""
        f = _h.H5Fopen(path.encode(), 0, 0)
        assert f >= 0, path
        d = _h.H5Dopen2(f, name.encode(), 0)
        assert d >= 0, name
        s, t = _h.H5Dget_space(d), _h.H5Dget_type(d)
        mem, dt = _mem(t)
        out = np.zeros(_dims(s), dtype=dt)
        if out.size:
            assert _h.H5Dread(d, mem, 0, 0, 0, out.ctypes.data_as(C.c_void_p)) >= 0
        _h.H5Tclose(t), _h.H5Sclose(s), _h.H5Dclose(d), _h.H5Fclose(f)
        return out

    def attr(path, obj, name):
        """Attribute -> (numpy array, shape tuple); shape () for a scalar attribute."""
        f = _h.H5Fopen(path.encode(), 0, 0)
        o = _h.H5Oopen(f, obj.encode(), 0)
        assert o >= 0, obj
        a = _h.H5Aopen_name(o, name.encode())
        assert a >= 0, name
        s, t = _h.H5Aget_space(a), _h.H5Aget_type(a)
        mem, dt = _mem(t)
        shape = _dims(s)
        out = np.zeros(shape if shape else (1,), dtype=dt)
        assert _h.H5Aread(a, mem, out.ctypes.data_as(C.c_void_p)) >= 0
        _h.H5Tclose(t), _h.H5Sclose(s), _h.H5Aclose(a), _h.H5Oclose(o), _h.H5Fclose(f)
        return out, shape

    def exists(path, name):
        f = _h.H5Fopen(path.encode(), 0, 0)
        parts, cur, ok = name.strip("/").split("/"), "", True
        for p in parts:
            cur = f"{cur}/{p}" if cur else p
            if _h.H5Lexists(f, cur.encode(), 0) <= 0:
                ok = False
                break
        _h.H5Fclose(f)
        return ok
