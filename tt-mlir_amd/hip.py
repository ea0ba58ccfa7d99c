"""ctypes binding of the gfx950 kernel library (include/ttmlir_amd_hip.h).

There is no fallback: if the shared library is missing, `lib()` raises.  Device buffers are
plain integer addresses (e.g. torch_tensor.data_ptr()); streams are raw hipStream_t handles.
"""
import ctypes
import os
import re

_HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(_HERE)
# TTMLIR_AMD_HIP_LIB names another build of the library (a kernel variant under measurement)
LIB_PATH = os.environ.get("TTMLIR_AMD_HIP_LIB") or os.path.join(_HERE, "lib", "libttmlir_amd_hip.so")
HEADER = os.path.join(ROOT, "include", "ttmlir_amd_hip.h")

F32, F16, BF16, BFP8B, BFP4B, U32, U16, U8, I32 = 0, 1, 2, 4, 6, 9, 10, 11, 12
ROW_MAJOR, TILE = 0, 1
ACT = {None: 0, "": 0, "gelu": 1, "silu": 2, "sigmoid": 3, "relu": 4}


class TTMError(RuntimeError):
    pass


_CTYPES = {
    "int": ctypes.c_int, "int64_t": ctypes.c_int64, "uint32_t": ctypes.c_uint32, "size_t": ctypes.c_size_t,
    "float": ctypes.c_float, "double": ctypes.c_double,
}


def declared_functions(header=HEADER):
    """[(name, restype, [argtypes])] parsed from the C header: the ABI contract."""
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = []
    for m in re.finditer(r"^\s*(const char \*|int64_t |int )\s*(ttm_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.M | re.S):
        ret, name, args = m.group(1).strip(), m.group(2), m.group(3)
        res = {"const char *": ctypes.c_char_p, "int64_t": ctypes.c_int64, "int": ctypes.c_int}[ret]
        argtypes = []
        for a in [x.strip() for x in args.replace("\n", " ").split(",")]:
            if a in ("void", ""):
                continue
            if "*" in a:
                if re.match(r"(const )?char \*", a) and "**" not in a and name != "ttm_device_name":
                    argtypes.append(ctypes.c_char_p)
                else:
                    argtypes.append(ctypes.c_void_p)
            else:
                argtypes.append(_CTYPES[a.rsplit(" ", 1)[0].replace("const ", "").strip()])
        out.append((name, res, argtypes))
    return out


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise TTMError("native kernel library missing: %s (run `python tt-mlir_amd/build.py`)" % LIB_PATH)
        l = ctypes.CDLL(LIB_PATH)
        for name, res, argtypes in declared_functions():
            fn = getattr(l, name)
            fn.restype, fn.argtypes = res, argtypes
        _lib = l
    return _lib


def check(status, what=""):
    if status != 0:
        msg = lib().ttm_last_error().decode()
        raise TTMError("%s failed (%d): %s" % (what or "ttm call", status, msg))


def call(name, *args):
    check(getattr(lib(), name)(*args), name)


def ptr(t):
    """Device address of a torch tensor (must be contiguous)."""
    assert t.is_contiguous()
    return ctypes.c_void_p(t.data_ptr())


def current_stream():
    """Raw hipStream_t of torch's current stream, so kernels order with torch work."""
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def set_option(name, value):
    call("ttm_set_option", name.encode(), int(value))


def get_option(name):
    v = ctypes.c_int(0)
    call("ttm_get_option", name.encode(), ctypes.byref(v))
    return v.value


def device_name():
    buf = ctypes.create_string_buffer(256)
    call("ttm_device_name", buf, 256)
    return buf.value.decode()


def bfp_tile_bytes(fmt):
    return int(lib().ttm_bfp_tile_bytes(fmt))


class Event:
    def __init__(self):
        self.h = ctypes.c_void_p()
        call("ttm_event_create", ctypes.byref(self.h))

    def record(self, stream=None):
        call("ttm_event_record", self.h, stream)

    def sync(self):
        call("ttm_event_sync", self.h)

    def elapsed_ms(self, stop):
        ms = ctypes.c_float()
        call("ttm_event_elapsed_ms", ctypes.byref(ms), self.h, stop.h)
        return ms.value

    def __del__(self):
        try:
            lib().ttm_event_destroy(self.h)
        except Exception:
            pass
