"""ctypes view of the C ABI declared in include/dmm.h (libdmm.so).

This is the stub a non-PyTorch host would write; the GPU parity tests call the kernels
through it with raw device pointers so that the boundary itself is what gets tested."""
import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libdmm.so")

# every symbol include/dmm.h declares: name -> (restype, argtypes)
_P, _I64, _F = ctypes.c_void_p, ctypes.c_int64, ctypes.c_float
_OP = [_P, _P, _P, _F, _P, _I64, _I64, _I64, _P]
SYMBOLS = {
    "dmm_version": (ctypes.c_int, []),
    "dmm_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "dmm_init": (ctypes.c_int, [ctypes.c_int]),
    "dmm_noalloc_scratch_bytes": (ctypes.c_int64, []),
    "dmm_decode_matmul_noalloc_f16": (ctypes.c_int, _OP),
    "dmm_decode_f16": (ctypes.c_int, [_P, _P, _P, _I64, _I64, _P]),
    "dmm_decode_matmul_f16": (ctypes.c_int, _OP),
    "dmm_gemv_f16": (ctypes.c_int, _OP),
    "dmm_gemv_8bit_f16": (ctypes.c_int, _OP),
    "dmm_gemv_kernel_name": (ctypes.c_char_p, [_I64, _I64, _I64]),
    "dmm_integer_kernel_name": (ctypes.c_char_p, [_I64, _I64, _I64]),
    "dmm_set_gemv_8bit": (ctypes.c_int, [ctypes.c_int]),
    "dmm_set_choice": (ctypes.c_int, [ctypes.c_int, ctypes.c_int]),
    "dmm_gemm_f16": (ctypes.c_int, _OP),
    "dmm_generic_f16": (ctypes.c_int, _OP),
    "dmm_workspace_bytes": (ctypes.c_int64, [_I64, _I64, _I64]),
    "dmm_decode_matmul_ws_f16": (ctypes.c_int, [_P, _P, _P, ctypes.c_float, _P, _I64, _I64, _I64, _P, _I64, _P]),
    "dmm_packed_bytes": (ctypes.c_int64, [_I64, _I64]),
    "dmm_pack_codes": (ctypes.c_int, [_P, _P, _I64, _I64, _P]),
    "dmm_gemv_packed_f16": (ctypes.c_int, _OP),
    "dmm_decode_matmul_packed_f16": (ctypes.c_int, [_P, _P, _P, ctypes.c_float, _P, _I64, _I64, _I64, _P, _I64, _P]),
    "dmm_decode_matmul_i8": (ctypes.c_int, [_P, _P, _P, _P, _I64, _I64, _I64, ctypes.c_int, _P]),
    "dmm_set_kernel_events": (ctypes.c_int, [_P, _P]),
    "dmm_decode_host_f16": (ctypes.c_int, [_P, _P, _P, _I64, _I64]),
    "dmm_decode_matmul_host_f16": (ctypes.c_int, [_P, _P, _P, _F, _P, _I64, _I64, _I64]),
    "dmm_read_probe": (ctypes.c_int, [_P, _P, _I64, _I64, _P]),
}

_lib = None


def lib():
    """The loaded library with argument types set.  Raises OSError if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OSError("libdmm.so is not built: run `python -m decode_matmul_amd.build`")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def status_string(status):
    return lib().dmm_status_string(int(status)).decode()


class DmmError(RuntimeError):
    def __init__(self, what, status):
        super().__init__("%s failed: %s (status %d)" % (what, status_string(status), status))
        self.status = status


def check(what, status):
    if status != 0:
        raise DmmError(what, status)
