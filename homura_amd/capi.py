"""ctypes binding of the C ABI in include/homura_rocm.h.

This is the thinnest possible caller of libhomura_rocm.so: the structs, the prototypes and a few
conveniences (contexts, device buffers, status -> exception). It is what the parity tests and
bench.py use to reach the kernels "through the C ABI"; it contains no arithmetic and no fallback:
if the shared library is missing, importing this module raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, byref, c_char, c_char_p, c_double, c_int32, c_int64, c_uint8, c_uint32, c_uint64, c_void_p

import numpy as np

HMR_OK, HMR_OUT_OF_MEMORY, HMR_INVALID, HMR_HIP_ERROR, HMR_INTERNAL_ERROR = range(5)
HMR_MAX_DIMS = 25
HMR_NAME_LEN, HMR_ARCH_LEN = 256, 64

# dtype codes (ref: csrc/homura_rocm.h:102-113)
BOOL, U8, I8, I16, I32, I64, F16, BF16, F32, F64 = range(10)
DTYPE_NAMES = ["bool", "u8", "i8", "i16", "i32", "i64", "f16", "bf16", "f32", "f64"]
DTYPE_SIZE = [1, 1, 1, 2, 4, 8, 2, 2, 4, 8]
# numpy storage type per dtype code (f16/bf16 travel as raw uint16 patterns, bool as uint8)
DTYPE_NP = [np.uint8, np.uint8, np.int8, np.int16, np.int32, np.int64, np.uint16, np.uint16, np.float32, np.float64]

UNARY = {n: i for i, n in enumerate(
    ["neg", "abs", "sign", "relu", "exp", "log", "sqrt", "rsqrt", "reciprocal", "sin", "cos", "erf", "tanh",
     "sigmoid", "log_sigmoid", "silu", "gelu", "gelu_tanh", "logical_not"])}
BINARY = {n: i for i, n in enumerate(
    ["add", "sub", "mul", "div", "pow", "maximum", "minimum", "greater", "greater_equal", "less", "less_equal",
     "equal", "not_equal", "logical_and", "logical_or", "bitwise_and"])}
REDUCE = {n: i for i, n in enumerate(["sum", "prod", "mean", "max", "min", "all", "any"])}


class hmr_device_properties(ctypes.Structure):
    _fields_ = [("name", c_char * HMR_NAME_LEN), ("arch", c_char * HMR_ARCH_LEN),
                ("multiprocessor_count", c_int32), ("warp_size", c_int32), ("total_memory", c_uint64)]


class hmr_tensor_desc(ctypes.Structure):
    _fields_ = [("data", c_void_p), ("offset", c_int64), ("dtype", c_int32), ("ndim", c_int32),
                ("sizes", c_int64 * HMR_MAX_DIMS), ("strides", c_int64 * HMR_MAX_DIMS)]


class hmr_abi_info(ctypes.Structure):
    _fields_ = [("abi_info_size", c_uint32), ("properties_size", c_uint32), ("properties_align", c_uint32),
                ("properties_offsets", c_uint32 * 5), ("status_values", c_int32 * 5), ("name_len", c_int32),
                ("arch_len", c_int32), ("desc_size", c_uint32), ("desc_align", c_uint32),
                ("desc_offsets", c_uint32 * 6), ("dtype_values", c_int32 * 10), ("max_dims", c_int32),
                ("gemm_desc_size", c_uint32), ("gemm_desc_align", c_uint32)]


DESC_P = POINTER(hmr_tensor_desc)
CTX = c_void_p

# name -> (restype, argtypes). Exactly the declarations of include/homura_rocm.h + _ext.h.
PROTOTYPES = {
    "hmr_last_error": (c_char_p, []),
    "hmr_device_count": (c_int32, [POINTER(c_int32)]),
    "hmr_device_properties_get": (c_int32, [c_int32, POINTER(hmr_device_properties)]),
    "hmr_mem_get_info": (c_int32, [c_int32, POINTER(c_uint64), POINTER(c_uint64)]),
    "hmr_context_create": (c_int32, [c_int32, POINTER(CTX)]),
    "hmr_context_destroy": (c_int32, [CTX]),
    "hmr_context_synchronize": (c_int32, [CTX]),
    "hmr_malloc": (c_int32, [c_int32, c_uint64, POINTER(c_void_p)]),
    "hmr_free": (c_int32, [c_int32, c_void_p]),
    "hmr_memset": (c_int32, [CTX, c_void_p, c_uint8, c_uint64]),
    "hmr_copy_to_host": (c_int32, [CTX, c_void_p, c_void_p, c_uint64]),
    "hmr_copy_from_host": (c_int32, [CTX, c_void_p, c_void_p, c_uint64]),
    "hmr_copy": (c_int32, [CTX, DESC_P, DESC_P]),
    "hmr_fill": (c_int32, [CTX, DESC_P, c_uint64]),
    "hmr_copy_device": (c_int32, [CTX, c_void_p, c_void_p, c_uint64]),
    "hmr_unary": (c_int32, [CTX, c_int32, DESC_P, DESC_P]),
    "hmr_binary": (c_int32, [CTX, c_int32, DESC_P, DESC_P, DESC_P]),
    "hmr_binary_constant": (c_int32, [CTX, c_int32, DESC_P, DESC_P, c_uint64, c_int32]),
    "hmr_binary_scalar": (c_int32, [CTX, c_int32, DESC_P, DESC_P, c_double, c_int32]),
    "hmr_where": (c_int32, [CTX, DESC_P, DESC_P, DESC_P, DESC_P]),
    "hmr_where_constant": (c_int32, [CTX, DESC_P, DESC_P, DESC_P, c_uint64, DESC_P, c_uint64]),
    "hmr_fused": (c_int32, [CTX, c_int32, DESC_P, DESC_P, DESC_P, DESC_P, c_double, c_int32]),
    "hmr_addr": (c_int32, [CTX, DESC_P, DESC_P, DESC_P, DESC_P, c_double, c_double, c_int64, c_int64]),
    "hmr_triangle": (c_int32, [CTX, DESC_P, DESC_P, c_int64, c_int32]),
    "hmr_flip": (c_int32, [CTX, DESC_P, DESC_P]),
    "hmr_reduce_workspace": (c_int32, [DESC_P, DESC_P, c_int32, POINTER(c_int64)]),
    "hmr_reduce": (c_int32, [CTX, c_int32, DESC_P, DESC_P, DESC_P, c_void_p, c_int64]),
    "hmr_reduce_static": (c_int32, [CTX, c_int32, DESC_P, DESC_P, DESC_P]),
    "hmr_var": (c_int32, [CTX, DESC_P, DESC_P, DESC_P, c_double, c_int32, c_void_p, c_int64]),
    "hmr_arg_reduce": (c_int32, [CTX, DESC_P, DESC_P, DESC_P, DESC_P, c_int32, c_void_p, c_int64]),
    "hmr_softmax_workspace": (c_int32, [DESC_P, c_int64, c_int64, POINTER(c_int64)]),
    "hmr_softmax": (c_int32, [CTX, DESC_P, DESC_P, c_int64, c_int64, c_int64, c_int32, c_void_p, c_int64]),
    "hmr_random_uniform": (c_int32, [CTX, DESC_P, c_uint64, c_uint64, c_double, c_double]),
    "hmr_random_normal": (c_int32, [CTX, DESC_P, c_uint64, c_uint64, c_double, c_double]),
    "hmr_random_int": (c_int32, [CTX, DESC_P, c_uint64, c_uint64, c_uint64, c_int64, c_uint64, c_uint64, c_void_p]),
    "hmr_index_check": (c_int32, [CTX, DESC_P, c_int64, c_int64, c_int32, c_int64, c_void_p]),
    "hmr_index_select": (c_int32, [CTX, DESC_P, DESC_P, DESC_P, c_int32, c_int32]),
    "hmr_gather": (c_int32, [CTX, DESC_P, DESC_P, DESC_P, c_int32]),
    "hmr_index_add_workspace": (c_int32, [c_int64, c_int64, POINTER(c_int64)]),
    "hmr_index_add": (c_int32, [CTX, DESC_P, DESC_P, DESC_P, c_int32, c_void_p, c_int64]),
    "hmr_scatter_add_workspace": (c_int32, [c_int64, POINTER(c_int64)]),
    "hmr_scatter_add": (c_int32, [CTX, DESC_P, DESC_P, DESC_P, c_int32, c_void_p, c_int64]),
    "hmr_index_positions": (c_int32, [CTX, DESC_P, DESC_P, c_int64, c_int64, c_int32]),
    "hmr_index_overwrite_workspace": (c_int32, [c_int64, POINTER(c_int64)]),
    "hmr_index_overwrite": (c_int32, [CTX, DESC_P, DESC_P, DESC_P, c_int32, c_void_p, c_int64]),
    "hmr_mask_workspace": (c_int32, [c_int64, POINTER(c_int64), POINTER(c_int64)]),
    "hmr_mask_count": (c_int32, [CTX, DESC_P, c_void_p, c_int64]),
    "hmr_mask_coordinates": (c_int32, [CTX, DESC_P, c_void_p, c_int64, DESC_P]),
    "hmr_exclusive_cumprod": (c_int32, [CTX, DESC_P, DESC_P, c_int64, c_int64, c_int64, c_int32]),
    "hmr_built_archs": (c_char_p, []),
    "hmr_abi_check": (None, [POINTER(hmr_abi_info)]),
    "hmr_test_fail_stream_create": (None, [c_int32]),
    "hmr_test_fail_after_probe": (None, [c_int32]),
    "hmr_test_fail_properties": (None, [c_int32]),
    "hmr_test_fail_data": (None, [c_int32, c_int32]),
    "hmr_test_reduce_plan": (c_int32, [DESC_P, DESC_P, POINTER(c_int64), POINTER(c_int64), POINTER(c_int64)]),
    "hmr_test_softmax_plan": (c_int32, [DESC_P, c_int64, c_int64, POINTER(c_int32), POINTER(c_int32),
                                        POINTER(c_int32)]),
    "hmr_test_index_value": (c_int32, [CTX, DESC_P, c_void_p]),
    "hmr_test_live_streams": (c_int32, []),
    "hmr_test_current_device": (c_int32, [POINTER(c_int32)]),
    "hmr_test_set_current_device": (c_int32, [c_int32]),
    "hmr_test_fail": (c_int32, [c_char_p]),
    "hmr_ext_stream": (c_int32, [CTX, POINTER(c_void_p)]),
}

# Exported stubs of other kernel families (include/homura_rocm_unbuilt.h); bound without prototypes.
UNBUILT = [
    "hmr_max_pool2d_backward_workspace", "hmr_max_pool2d_backward", "hmr_max_pool2d",
    "hmr_max_pool2d_check", "hmr_max_pool2d_gather_backward", "hmr_adaptive_avg_pool2d",
    "hmr_adaptive_avg_pool2d_backward", "hmr_unfold_backward", "hmr_gemm_fold", "hmr_gemm_select",
    "hmr_gemm_path_name", "hmr_gemm_workspace", "hmr_gemm", "hmr_test_wide_pool",
    "hmr_test_force_gemm_path", "hmr_test_pool_candidates",
]

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libhomura_rocm.so")


class HmrError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"hmr status {status}: {message}")
        self.status = status
        self.message = message


def load(path: str = LIB_PATH) -> ctypes.CDLL:
    """Loads libhomura_rocm.so and declares every prototype. Raises if the library is absent."""
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or `make -C homura_amd/csrc`). There is no fallback implementation.")
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


lib = load()


def check(status: int) -> None:
    if status != HMR_OK:
        raise HmrError(status, lib.hmr_last_error().decode("utf-8", "replace"))


def make_desc(ptr: int, dtype: int, sizes=(), strides=(), offset: int = 0) -> hmr_tensor_desc:
    d = hmr_tensor_desc()
    d.data = ptr
    d.offset = offset
    d.dtype = dtype
    d.ndim = len(sizes)
    for i, (n, s) in enumerate(zip(sizes, strides)):
        d.sizes[i] = n
        d.strides[i] = s
    return d


class Context:
    """One device's execution context (its stream)."""

    def __init__(self, device: int = 0):
        self.device = device
        self.handle = CTX()
        check(lib.hmr_context_create(device, byref(self.handle)))

    def close(self) -> None:
        if self.handle:
            check(lib.hmr_context_destroy(self.handle))
            self.handle = CTX()

    def synchronize(self) -> None:
        check(lib.hmr_context_synchronize(self.handle))

    def stream(self) -> int:
        s = c_void_p()
        check(lib.hmr_ext_stream(self.handle, byref(s)))
        return s.value or 0

    def malloc(self, nbytes: int) -> "DeviceBuffer":
        return DeviceBuffer(self, nbytes)

    def upload(self, array: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(array)
        buf = DeviceBuffer(self, max(a.nbytes, 1))
        if a.nbytes:
            check(lib.hmr_copy_from_host(self.handle, buf.ptr, a.ctypes.data, a.nbytes))
        return buf


class DeviceBuffer:
    def __init__(self, ctx: Context, nbytes: int):
        self.ctx = ctx
        self.nbytes = nbytes
        p = c_void_p()
        check(lib.hmr_malloc(ctx.device, max(nbytes, 1), byref(p)))
        self.ptr = p.value

    def download(self, np_dtype, count: int) -> np.ndarray:
        out = np.empty(count, dtype=np_dtype)
        if out.nbytes:
            check(lib.hmr_copy_to_host(self.ctx.handle, out.ctypes.data, self.ptr, out.nbytes))
        return out

    def free(self) -> None:
        if self.ptr:
            check(lib.hmr_free(self.ctx.device, self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
