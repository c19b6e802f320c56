"""ctypes access to the CPU oracle (oracle/liboracle.so). Test infrastructure only."""
import ctypes
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "oracle", "liboracle.so")


class hcb_tensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("offset", ctypes.c_int64), ("dtype", ctypes.c_int32),
                ("ndim", ctypes.c_int32), ("shape", ctypes.POINTER(ctypes.c_int64)),
                ("strides", ctypes.POINTER(ctypes.c_int64))]


class hcb_scalar(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("reserved", ctypes.c_int32), ("i", ctypes.c_int64), ("f", ctypes.c_double)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
        _lib = ctypes.CDLL(LIB)
        _lib.orc_backend.restype = ctypes.c_void_p
        _lib.orc_last_error.restype = ctypes.c_char_p
        _lib.orc_erf.restype = ctypes.c_double
        _lib.orc_erf.argtypes = [ctypes.c_double]
        _lib.orc_int_pow_i64.restype = ctypes.c_int64
        _lib.orc_int_pow_i64.argtypes = [ctypes.c_int64, ctypes.c_int64]
        _lib.orc_int_pow_i32.restype = ctypes.c_int32
        _lib.orc_int_pow_i32.argtypes = [ctypes.c_int32, ctypes.c_int32]
        _lib.orc_int_pow_i8.restype = ctypes.c_int8
        _lib.orc_int_pow_i8.argtypes = [ctypes.c_int8, ctypes.c_int8]
    return _lib


def backend_address() -> int:
    """Address of the oracle's hcb_backend table, for _host.register_cpu_backend."""
    return lib().orc_backend()


def tensor(array, dtype_code, shape=None, strides=None, offset=0):
    """An hcb_tensor over a numpy array's memory (the array must stay alive)."""
    shape = list(array.shape if shape is None else shape)
    if strides is None:
        strides, s = [], 1
        for n in reversed(shape):
            strides.insert(0, s)
            s *= n
    t = hcb_tensor()
    t.data = array.ctypes.data
    t.offset = offset
    t.dtype = dtype_code
    t.ndim = len(shape)
    t._shape = (ctypes.c_int64 * max(len(shape), 1))(*shape)
    t._strides = (ctypes.c_int64 * max(len(shape), 1))(*strides)
    t.shape = ctypes.cast(t._shape, ctypes.POINTER(ctypes.c_int64))
    t.strides = ctypes.cast(t._strides, ctypes.POINTER(ctypes.c_int64))
    return t


def check(rc):
    if rc != 0:
        raise RuntimeError(lib().orc_last_error().decode())
