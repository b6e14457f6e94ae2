"""Loader of libarkmi.so and the ctypes signatures of its C ABI."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libarkmi.so")
_lib = None

DTYPES = {"fp32": 0, "fp16": 1, "bf16": 2, "int32": 3, "uint32": 4, "int8": 5,
          "uint8": 6, "byte": 7}

_STATUS_NAMES = {1: "InternalError", 2: "InvalidUsageError", 3: "ModelError",
                 4: "PlanError", 5: "UnsupportedError", 6: "SystemError",
                 7: "GpuError"}


class ArkmiError(RuntimeError):
    """Base of the error classes (ark::BaseError, ark/include/ark/error.hpp:13-43).
    Raised by check() for a non-zero status from the C ABI: `.code` is the
    arkmi_status value and `.kind` the name of the matching ark:: error class,
    and the object is an instance of the subclass of that name.  Raised from
    Python with a message alone, str() is that message."""
    code = 0

    def __init__(self, *args):
        if len(args) == 2 and isinstance(args[0], int):
            self.code = args[0]
            self.kind = _STATUS_NAMES.get(args[0], "Error")
            super().__init__(f"{self.kind}: {args[1]}")
        else:
            self.kind = _STATUS_NAMES.get(self.code, "Error")
            super().__init__(*args)


BaseError = ArkmiError


def _error_class(code, name):
    return type(name, (ArkmiError,), {"code": code, "__doc__": f"ark::{name}"})


InternalError = _error_class(1, "InternalError")
InvalidUsageError = _error_class(2, "InvalidUsageError")
ModelError = _error_class(3, "ModelError")
PlanError = _error_class(4, "PlanError")
UnsupportedError = _error_class(5, "UnsupportedError")
SystemError = _error_class(6, "SystemError")  # noqa: A001 (the reference's name)
GpuError = _error_class(7, "GpuError")
_ERROR_CLASSES = {c.code: c for c in (InternalError, InvalidUsageError, ModelError, PlanError,
                                      UnsupportedError, SystemError, GpuError)}


class DeviceInfo(ctypes.Structure):
    _fields_ = [("device_id", ctypes.c_int), ("num_cu", ctypes.c_int),
                ("wave_size", ctypes.c_int), ("max_threads_per_block", ctypes.c_int),
                ("lds_bytes_per_cu", ctypes.c_int), ("l2_bytes", ctypes.c_int),
                ("hbm_bytes", ctypes.c_size_t), ("clock_khz", ctypes.c_int),
                ("arch", ctypes.c_char * 32), ("gcn_arch", ctypes.c_char * 64)]


def lib():
    """The loaded native library.  There is no fallback: a missing library is
    an error, so nothing can silently run without the HIP path."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise ImportError(
                f"{_LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C ark_amd/csrc`")
        L = ctypes.CDLL(_LIB_PATH)
        L.arkmi_last_error.restype = ctypes.c_char_p
        L.arkmi_version.restype = ctypes.c_char_p
        L.arkmi_free.argtypes = [ctypes.c_void_p]
        L.arkmi_free.restype = None
        _lib = L
    return _lib


def check(status):
    if status != 0:
        raise _ERROR_CLASSES.get(status, ArkmiError)(
            status, lib().arkmi_last_error().decode(errors="replace"))


def device_info(device_id=0):
    info = DeviceInfo()
    check(lib().arkmi_device_info_get(ctypes.c_int(device_id), ctypes.byref(info)))
    return {f: (getattr(info, f).decode() if isinstance(getattr(info, f), bytes)
                else getattr(info, f)) for f, _ in DeviceInfo._fields_}
