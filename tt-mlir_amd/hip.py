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
        if _check_buffers:   # switched on by the environment before the library was loaded: the library's own check goes with it
            l.ttm_set_option(b"check_extents", 1)
    return _lib


def check(status, what=""):
    if status != 0:
        msg = lib().ttm_last_error().decode()
        raise TTMError("%s failed (%d): %s" % (what or "ttm call", status, msg))


class _Ptr(ctypes.c_void_p):
    """A device address that remembers how many bytes follow it in its tensor."""
    nbytes = None


_ELEM_BYTES = {F32: 4, F16: 2, BF16: 2, U32: 4, U16: 2, U8: 1, I32: 4}


def _pad32(n):
    return (int(n) + 31) // 32 * 32


def _tile_bytes(batch, rows, cols, elem):
    return int(batch) * _pad32(rows) * _pad32(cols) * elem


def _plain_bytes(batch, rows, cols, elem):
    return int(batch) * int(rows) * int(cols) * elem


def _vec_bytes(layout, cols, elem):   # a [cols] weight / bias vector: one tile row of 32 rows, or the plain vector
    return 32 * _pad32(cols) * elem if layout == TILE else int(cols) * elem


# The entry points take logical extents and no buffer sizes; a tile tensor must be backed by its whole padded extent.
# Per entry point: (argument index, bytes the kernels touch from that pointer on, what it is).
_EXTENTS = {
    "ttm_tilize": lambda a: [(0, _plain_bytes(a[2], a[3], a[4], a[5]), "row-major input"), (1, _tile_bytes(a[2], a[3], a[4], a[5]), "tile output")],
    "ttm_untilize": lambda a: [(0, _tile_bytes(a[2], a[3], a[4], a[5]), "tile input"), (1, _plain_bytes(a[2], a[3], a[4], a[5]), "row-major output")],
    "ttm_softmax_lastdim": lambda a: [(i, _tile_bytes(a[3], a[4], a[5], _ELEM_BYTES[a[2]]), w) for i, w in ((0, "tile input"), (1, "tile output"))],
    "ttm_reduce_lastdim": lambda a: [(1, _tile_bytes(a[4], a[5], a[6], _ELEM_BYTES[a[3]]), "tile input"),
                                     (2, _tile_bytes(a[4], a[5], 1, _ELEM_BYTES[a[3]]), "tile output [.., rows, 1]")],
    "ttm_rms_norm": lambda a: [(0, _tile_bytes(a[7], a[8], a[9], _ELEM_BYTES[a[6]]), "tile input"),
                               (1, _vec_bytes(a[2], a[9], _ELEM_BYTES[a[6]]), "weight"), (3, _vec_bytes(a[4], a[9], _ELEM_BYTES[a[6]]), "bias"),
                               (5, _tile_bytes(a[7], a[8], a[9], _ELEM_BYTES[a[6]]), "tile output")],
    "ttm_eltwise_unary": lambda a: [(i, (_tile_bytes if a[4] == TILE else _plain_bytes)(a[5], a[6], a[7], _ELEM_BYTES[a[3]]), w)
                                    for i, w in ((1, "input"), (2, "output"))],
}


def _tiles(batch, rows, cols):
    return int(batch) * (_pad32(rows) // 32) * (_pad32(cols) // 32)


def _operand_bytes(dtype, batch, rows, cols):   # a tile tensor of a plain or block-float dtype
    if dtype in (BFP8B, BFP4B):
        return _tiles(batch, rows, cols) * (1088 if dtype == BFP8B else 576)
    return _tile_bytes(batch, rows, cols, _ELEM_BYTES[dtype])


_EXTENTS.update({
    # (src, src_dtype, src_layout, dst, fmt, batch, rows, cols)
    "ttm_bfp_pack": lambda a: [(0, (_tile_bytes if a[2] == TILE else _plain_bytes)(a[5], a[6], a[7], _ELEM_BYTES[a[1]]), "input"),
                               (3, _operand_bytes(a[4], a[5], a[6], a[7]), "block-float output")],
    # (src, fmt, dst, dst_dtype, dst_layout, batch, rows, cols)
    "ttm_bfp_unpack": lambda a: [(0, _operand_bytes(a[1], a[5], a[6], a[7]), "block-float input"),
                                 (2, (_tile_bytes if a[4] == TILE else _plain_bytes)(a[5], a[6], a[7], _ELEM_BYTES[a[3]]), "output")],
    # (a, a_dtype, w, w_dtype, transpose_w, bias, bias_dtype, bias_layout, out, out_dtype, batch, w_batch, M, N, K, act)
    "ttm_linear": lambda a: [(0, _operand_bytes(a[1], a[10], a[12], a[14]), "activations [batch, M, K]"),
                             (2, _operand_bytes(a[3], a[11], a[14], a[13]), "weights [w_batch, K, N]"),
                             (5, _vec_bytes(a[7], a[13], _ELEM_BYTES[a[6]]), "bias"),
                             (8, _operand_bytes(a[9], a[10], a[12], a[13]), "output [batch, M, N]")],
    # (in, src_dtype, out, dst_dtype, n)
    "ttm_typecast": lambda a: [(0, int(a[4]) * _ELEM_BYTES[a[1]], "input"), (2, int(a[4]) * _ELEM_BYTES[a[3]], "output")],
    "ttm_copy_kernel": lambda a: [(0, int(a[2]), "source"), (1, int(a[2]), "destination")],
    # (in, dtype, out, rows, cols): row-major on both sides
    "ttm_argmax": lambda a: [(0, int(a[3]) * int(a[4]) * _ELEM_BYTES[a[1]], "input"), (2, int(a[3]) * 4, "int32 output")],
})
_check_buffers = os.environ.get("TTMLIR_AMD_CHECK_BUFFERS", "0") == "1"


def check_buffers(on=True):
    """Switch the host-side check of buffer extents on or off (TTMLIR_AMD_CHECK_BUFFERS=1 switches it on at import): before a
    call of one of the entry points listed in _EXTENTS, every pointer made by ptr() must have at least the bytes behind it
    that the kernels will touch.  A kernel that runs past a buffer faults the whole device, so the check belongs in front
    of any call whose buffers were sized by hand."""
    global _check_buffers
    _check_buffers = bool(on)
    # the library's own check covers every entry point (the rules above cover the common ones, against the tensor's size,
    # which is tighter than the allocation the library can see)
    set_option("check_extents", 1 if on else 0)


def _verify_extents(name, args):
    spec = _EXTENTS.get(name)
    if spec is None:
        return
    try:
        extents = spec(args)
    except (KeyError, IndexError, TypeError) as e:
        # arguments the size rules here do not cover (an unknown dtype code, a short argument list): the library's own check,
        # which is on whenever this one is and holds every operand of every entry point against its allocation, answers;
        # without it the call is refused rather than let through unchecked
        v = ctypes.c_int(0)
        lib().ttm_get_option(b"check_extents", ctypes.byref(v))
        if v.value == 1:
            return
        raise TTMError("%s: buffer extents cannot be checked for these arguments (%s: %s)" % (name, type(e).__name__, e))
    for idx, need, what in extents:
        p = args[idx]
        if isinstance(p, _Ptr) and p.nbytes is not None and p.nbytes < need:
            raise TTMError("%s: the %s (argument %d) has %d bytes, the kernels touch %d from its address on (tile tensors are "
                           "padded to whole 32 x 32 tiles)" % (name, what, idx, p.nbytes, need))


def call(name, *args):
    if _check_buffers:
        _verify_extents(name, args)
    check(getattr(lib(), name)(*args), name)


def ptr(t):
    """Device address of a torch tensor (must be contiguous); it carries the tensor's size for check_buffers."""
    assert t.is_contiguous()
    p = _Ptr(t.data_ptr())
    p.nbytes = t.numel() * t.element_size()
    return p


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
