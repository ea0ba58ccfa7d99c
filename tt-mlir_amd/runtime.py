"""Python surface of the host runtime (ctypes over lib/libttmlir_amd_rt.so).

Mirrors the calls a tt-mlir harness makes on `ttrt.runtime` / `_ttmlir_runtime`
(tools/builder/base/builder_runtime.py:112-169, 694-803; tools/ttrt/common/run.py:534-873):
load a binary, open a device, create host tensors, get_layout / to_layout, submit, wait, to_host,
memcpy.  Tensors cross the boundary as numpy arrays (bf16 as uint16 bit patterns or torch tensors).
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libttmlir_amd_rt.so")
HEADER = os.path.join(os.path.dirname(_HERE), "include", "ttmlir_amd_runtime.h")


class RuntimeError_(RuntimeError):
    pass


class DataType:
    Float32, Float16, BFloat16, BFP_Float8, BFP_BFloat8, BFP_Float4, BFP_BFloat4, BFP_Float2, BFP_BFloat2 = range(9)
    UInt32, UInt16, UInt8, Int32, Float64, Int64, UInt64, Int16, Int8, Bool = range(9, 19)


class TensorLayout:
    RowMajor, Tile = 0, 1


class StorageType:
    Host, Device = 0, 1


class Layout(ctypes.Structure):
    _fields_ = [("storage", ctypes.c_int), ("layout", ctypes.c_int), ("dtype", ctypes.c_int)]

    def __repr__(self):
        return "Layout(storage=%d, layout=%d, dtype=%d)" % (self.storage, self.layout, self.dtype)

    def __eq__(self, o):
        return (self.storage, self.layout, self.dtype) == (o.storage, o.layout, o.dtype)


_NP_DTYPE = {DataType.Float32: np.float32, DataType.Float16: np.float16, DataType.BFloat16: np.uint16, DataType.UInt32: np.uint32,
             DataType.UInt16: np.uint16, DataType.UInt8: np.uint8, DataType.Int32: np.int32, DataType.Float64: np.float64,
             DataType.Int64: np.int64, DataType.UInt64: np.uint64, DataType.Int16: np.int16, DataType.Int8: np.int8,
             DataType.Bool: np.bool_}
_ITEMSIZE = {k: np.dtype(v).itemsize for k, v in _NP_DTYPE.items()}

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError_("native runtime library missing: %s (run `python tt-mlir_amd/build.py`)" % LIB_PATH)
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.ttrt_last_error.restype = ctypes.c_char_p
    return _lib


def declared_functions():
    import re
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ttrt_\w+)\s*\(", text)) - {"ttrt_op_callback"})


def _ck(status, what):
    if status != 0:
        raise RuntimeError_("%s: %s" % (what, lib().ttrt_last_error().decode("utf-8", "replace")))


def _call(name, *args):
    _ck(getattr(lib(), name)(*args), name)


def _shape_arg(shape):
    arr = (ctypes.c_uint32 * 8)(*[int(s) for s in shape])
    return arr, len(shape)


class Binary:
    def __init__(self, handle):
        self.h = handle

    @staticmethod
    def load_from_path(path):
        h = ctypes.c_void_p()
        _call("ttrt_binary_load_file", str(path).encode(), ctypes.byref(h))
        return Binary(h)

    @staticmethod
    def load_from_memory(data):
        h = ctypes.c_void_p()
        buf = (ctypes.c_uint8 * len(data)).from_buffer_copy(data)
        _call("ttrt_binary_load_memory", buf, ctypes.c_size_t(len(data)), ctypes.byref(h))
        return Binary(h)

    def store(self, path):
        _call("ttrt_binary_store", self.h, str(path).encode())

    def get_num_programs(self):
        n = ctypes.c_uint32()
        _call("ttrt_binary_num_programs", self.h, ctypes.byref(n))
        return n.value

    def get_program_name(self, i):
        buf = ctypes.create_string_buffer(256)
        _call("ttrt_binary_program_name", self.h, i, buf, 256)
        return buf.value.decode("utf-8", "replace")

    def is_program_private(self, i):
        v = ctypes.c_int()
        _call("ttrt_binary_program_is_private", self.h, i, ctypes.byref(v))
        return bool(v.value)

    def _descs(self, program, is_output):
        n = ctypes.c_uint32()
        _call("ttrt_binary_num_outputs" if is_output else "ttrt_binary_num_inputs", self.h, program, ctypes.byref(n))
        out = []
        for i in range(n.value):
            shape, rank, lay = (ctypes.c_uint32 * 8)(), ctypes.c_int(), Layout()
            _call("ttrt_binary_tensor_desc", self.h, program, int(is_output), i, shape, ctypes.byref(rank), ctypes.byref(lay))
            out.append((tuple(shape[: rank.value]), lay))
        return out

    def get_program_inputs(self, program):
        return self._descs(program, False)

    def get_program_outputs(self, program):
        return self._descs(program, True)

    def get_program_ops_as_text(self, program):
        buf = ctypes.create_string_buffer(1 << 16)
        _call("ttrt_binary_ops_text", self.h, program, buf, 1 << 16)
        return buf.value.decode("utf-8", "replace")

    def _json(self, program, which):
        import json
        need = ctypes.c_size_t()
        _call("ttrt_binary_program_json", self.h, program, which, None, 0, ctypes.byref(need))
        buf = ctypes.create_string_buffer(need.value + 1)
        _call("ttrt_binary_program_json", self.h, program, which, buf, need.value + 1, None)
        return json.loads(buf.value.decode("utf-8", "replace"))

    def get_program_inputs_as_json(self, program):
        """Parsed JSON view of the program's input TensorRefs (Binary.getProgramInputsAsJson)."""
        return self._json(program, 0)

    def get_program_outputs_as_json(self, program):
        return self._json(program, 1)

    def get_program_ops_as_json(self, program):
        """[{type_type, debug_info, loc_info}, ...] (Binary.getProgramOpsAsJson)."""
        return self._json(program, 2)

    def get_debug_info_golden(self, loc):
        """Embedded golden tensor for an op location as (name, numpy array) or None (Binary.getDebugInfoGolden).
        bf16 goldens come back as float32 values."""
        import numpy as np
        found, rank, dtype = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        shape = (ctypes.c_int64 * 8)()
        data, size = ctypes.POINTER(ctypes.c_uint8)(), ctypes.c_size_t()
        name = ctypes.create_string_buffer(256)
        _call("ttrt_binary_golden", self.h, loc.encode(), ctypes.byref(found), shape, ctypes.byref(rank), ctypes.byref(dtype),
              ctypes.byref(data), ctypes.byref(size), name, 256)
        if not found.value:
            return None
        raw = np.ctypeslib.as_array(data, shape=(size.value,)).copy()
        shp = tuple(shape[: rank.value])
        if dtype.value == DataType.BFloat16:
            arr = (raw.view(np.uint16).astype(np.uint32) << 16).view(np.float32).reshape(shp)
        else:
            arr = raw.view(_NP_DTYPE[dtype.value]).reshape(shp)
        return name.value.decode("utf-8", "replace"), arr

    def info(self):
        ident, ver = ctypes.create_string_buffer(5), ctypes.create_string_buffer(64)
        _call("ttrt_binary_info", self.h, ident, ver, 64)
        return ident.value.decode("utf-8", "replace"), ver.value.decode("utf-8", "replace")

    def __del__(self):
        try:
            lib().ttrt_binary_free(self.h)
        except Exception:
            pass


class Device:
    def __init__(self, handle):
        self.h = handle

    def name(self):
        buf = ctypes.create_string_buffer(256)
        _call("ttrt_device_name", self.h, buf, 256)
        return buf.value.decode("utf-8", "replace")


class Tensor:
    def __init__(self, handle, keepalive=None):
        self.h = handle
        self._keepalive = keepalive  # borrowed host memory must outlive the tensor

    def desc(self):
        shape, rank, lay, nbytes = (ctypes.c_uint32 * 8)(), ctypes.c_int(), Layout(), ctypes.c_uint64()
        _call("ttrt_tensor_desc", self.h, shape, ctypes.byref(rank), ctypes.byref(lay), ctypes.byref(nbytes))
        return tuple(shape[: rank.value]), lay, nbytes.value

    @property
    def shape(self):
        return self.desc()[0]

    @property
    def layout(self):
        return self.desc()[1]

    def is_allocated(self):
        v = ctypes.c_int()
        _call("ttrt_tensor_is_allocated", self.h, ctypes.byref(v))
        return bool(v.value)

    # the accessors of the reference's Tensor binding (runtime/python/runtime/runtime.cpp:213-262)
    def get_shape(self):
        return list(self.desc()[0])

    def get_layout(self):
        return self.desc()[1]

    def get_dtype(self):
        return self.desc()[1].dtype

    def has_layout(self, layout):
        v = ctypes.c_int()
        _call("ttrt_tensor_has_layout", self.h, ctypes.byref(layout), ctypes.byref(v))
        return bool(v.value)

    def _extent(self):
        vol, lvol, esz, stride = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint32(), (ctypes.c_int64 * 8)()
        _call("ttrt_tensor_extent", self.h, ctypes.byref(vol), ctypes.byref(lvol), ctypes.byref(esz), stride)
        return vol.value, lvol.value, esz.value, list(stride[: len(self.desc()[0])])

    def get_volume(self):
        """Elements in storage: the tile layout's padding counts."""
        return self._extent()[0]

    def get_logical_volume(self):
        return self._extent()[1]

    def get_element_size(self):
        return self._extent()[2]

    def get_stride(self):
        return self._extent()[3]

    def get_tensor_desc(self):
        """shape / stride / dtype / item_size in one object, as the reference's TensorDesc binding has them."""
        import types
        return types.SimpleNamespace(shape=self.get_shape(), stride=self.get_stride(), dtype=self.get_dtype(),
                                     item_size=self.get_element_size())

    def get_data_buffer(self):
        """The tensor's bytes, read back and untilized if it lives on the device (getTensorDataBuffer)."""
        return bytearray(to_numpy(self).tobytes())

    def set_retain(self, retain):
        _call("ttrt_tensor_set_retain", self.h, int(retain))

    def get_retain(self):
        v = ctypes.c_int()
        _call("ttrt_tensor_get_retain", self.h, ctypes.byref(v))
        return bool(v.value)

    def __del__(self):
        try:
            lib().ttrt_tensor_free(self.h)
        except Exception:
            pass


def get_num_available_devices():
    n = ctypes.c_uint32()
    _call("ttrt_num_devices", ctypes.byref(n))
    return n.value


def open_mesh_device():
    h = ctypes.c_void_p()
    _call("ttrt_device_open", ctypes.byref(h))
    return Device(h)


def close_mesh_device(dev):
    _call("ttrt_device_close", dev.h)
    dev.h = None


def _host(array, dtype, borrowed, stride=None):
    a = np.asarray(array)
    if stride is None:
        a = np.ascontiguousarray(a)
    shape, rank = _shape_arg(a.shape)
    st = None
    if stride is not None:
        st = (ctypes.c_int64 * 8)(*[int(s) for s in stride])
    h = ctypes.c_void_p()
    _call("ttrt_tensor_create_host", ctypes.c_void_p(a.ctypes.data), shape, rank, st, a.dtype.itemsize, dtype, int(borrowed),
          ctypes.byref(h))
    return Tensor(h, keepalive=a if borrowed else None)


def create_owned_host_tensor(array, dtype, stride=None):
    """createOwnedHostTensor: copies (and gathers strides); `array` is numpy, bf16 as uint16 bits."""
    return _host(array, dtype, False, stride)


def create_borrowed_host_tensor(array, dtype):
    """createBorrowedHostTensor: aliases the numpy buffer, which the returned object keeps alive."""
    return _host(array, dtype, True)


def from_torch(t, borrowed=False):
    """Host tensor from a CPU torch tensor (bf16 / f32 / f16 / ints)."""
    import torch
    m = {torch.float32: (DataType.Float32, None), torch.bfloat16: (DataType.BFloat16, torch.int16),
         torch.float16: (DataType.Float16, None), torch.int32: (DataType.Int32, None), torch.int64: (DataType.Int64, None),
         torch.uint8: (DataType.UInt8, None), torch.float64: (DataType.Float64, None), torch.int16: (DataType.Int16, None),
         torch.int8: (DataType.Int8, None), torch.bool: (DataType.Bool, None)}
    dt, view = m[t.dtype]
    a = t.contiguous()
    arr = a.view(view).numpy().view(np.uint16) if view is not None else a.numpy()
    return _host(arr, dt, borrowed)


def create_unsafe_borrowed_host_tensor(owned):
    """A borrowed Tensor over the buffer of an owned row-major host Tensor, no copy (createUnsafeBorrowedHostTensor); the
    returned object keeps `owned` alive, which is what the C++ caller has to see to itself."""
    h = ctypes.c_void_p()
    _call("ttrt_tensor_create_unsafe_borrowed", owned.h, ctypes.byref(h))
    return Tensor(h, keepalive=owned)


def host_data_ptr(tensor):
    """Address of a host tensor's buffer, 0 once it is deallocated."""
    p = ctypes.c_void_p()
    _call("ttrt_tensor_host_data", tensor.h, ctypes.byref(p))
    return p.value or 0


def create_empty_tensor(device, layout, shape):
    """Uninitialised tensor in `layout` (createEmptyTensor); `device` may be None for host storage."""
    sh, rank = _shape_arg(shape)
    h = ctypes.c_void_p()
    _call("ttrt_tensor_create_empty", device.h if device is not None else None, ctypes.byref(layout), sh, rank, ctypes.byref(h))
    return Tensor(h)


def dump_tensor(tensor, file_path):
    """Write the tensor to a file in its own layout (dumpTensor)."""
    _call("ttrt_tensor_dump", tensor.h, os.fsencode(file_path))


def load_tensor(file_path, device=None):
    """Read a tensor written by dump_tensor; on the host, or on `device` when one is given (loadTensor)."""
    h = ctypes.c_void_p()
    _call("ttrt_tensor_load", os.fsencode(file_path), device.h if device is not None else None, ctypes.byref(h))
    return Tensor(h)


def get_layout(binary, program, input_index):
    lay = Layout()
    _call("ttrt_get_layout", binary.h, program, input_index, ctypes.byref(lay))
    return lay


def to_layout(tensor, device, layout, retain=None):
    h = ctypes.c_void_p()
    _call("ttrt_to_layout", tensor.h, device.h, ctypes.byref(layout), -1 if retain is None else int(retain), ctypes.byref(h))
    return Tensor(h, keepalive=tensor._keepalive)


def to_host(tensor, untilize=False):
    h = ctypes.c_void_p()
    _call("ttrt_to_host", tensor.h, int(untilize), ctypes.byref(h))
    return [Tensor(h)]


def wait(tensor_or_list):
    for t in (tensor_or_list if isinstance(tensor_or_list, (list, tuple)) else [tensor_or_list]):
        _call("ttrt_wait", t.h)


def submit(device, binary, program, inputs):
    ins = (ctypes.c_void_p * max(1, len(inputs)))(*[t.h for t in inputs])
    outs = (ctypes.c_void_p * 64)()
    n = ctypes.c_uint32()
    del _callback_error[:]
    try:
        _call("ttrt_submit", device.h, binary.h, program, ins, len(inputs), outs, 64, ctypes.byref(n))
    except RuntimeError_:
        _raise_callback_error()   # the callback's own exception says more than what it led to
        raise
    results = [Tensor(ctypes.c_void_p(outs[i])) for i in range(n.value)]
    _raise_callback_error()
    return results


def deallocate_tensor(tensor, force=False):
    _call("ttrt_tensor_deallocate", tensor.h, int(force))


def memcpy(dst_array, src_tensor, target_dtype=None):
    """memcpy(void*, Tensor, optional<DataType>) into a numpy array."""
    _call("ttrt_memcpy_out", ctypes.c_void_p(dst_array.ctypes.data), src_tensor.h, -1 if target_dtype is None else target_dtype)


def memcpy_tensor(dst_tensor, src_tensor):
    """memcpy(Tensor, Tensor): the payload of src into dst, same size and data type."""
    _call("ttrt_memcpy_tensor", dst_tensor.h, src_tensor.h)


def to_numpy(tensor, target_dtype=None):
    """Host tensor -> numpy array (bf16 as uint16 bits; block-float host tensors as raw bytes)."""
    shape, lay, nbytes = tensor.desc()
    if lay.storage != StorageType.Host:
        tensor = to_host(tensor, untilize=True)[0]
        shape, lay, nbytes = tensor.desc()
    dt = lay.dtype if target_dtype is None else target_dtype
    if dt not in _NP_DTYPE or lay.layout == TensorLayout.Tile:
        out = np.empty(nbytes, dtype=np.uint8)
        memcpy(out, tensor)
        return out
    out = np.empty(shape, dtype=_NP_DTYPE[dt])
    memcpy(out, tensor, target_dtype)
    return out


def to_torch(tensor):
    import torch
    a = to_numpy(tensor)
    lay = tensor.desc()[1]
    if lay.dtype == DataType.BFloat16:
        return torch.from_numpy(a.view(np.int16)).view(torch.bfloat16)
    return torch.from_numpy(a)


def buffer_cast(src, from_dtype, to_dtype):
    src = np.ascontiguousarray(src)
    dst = np.empty(src.shape, dtype=_NP_DTYPE[to_dtype])
    _call("ttrt_buffer_cast", ctypes.c_void_p(src.ctypes.data), ctypes.c_void_p(dst.ctypes.data), from_dtype, to_dtype, ctypes.c_int64(src.size))
    return dst


def get_stat(name):
    v = ctypes.c_int64()
    _call("ttrt_stat", name.encode(), ctypes.byref(v))
    return v.value


def clear_stats():
    _call("ttrt_stats_clear")


_CB_TYPE = ctypes.CFUNCTYPE(None, ctypes.c_uint32, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_void_p, ctypes.c_void_p)
_PROGRAM_CB_TYPE = ctypes.CFUNCTYPE(None, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_void_p)
_cb_keep = {}


class HookContext:
    """What a callback may ask about the operation / program it runs for; valid only inside the callback.
    Calling the object returns the op's first output (kept for callbacks written as get_output())."""

    def __init__(self, hook):
        self._h = ctypes.c_void_p(hook)

    def output(self):
        """First output of the op as an untilized host Tensor, or None (getOpOutputTensor)."""
        h = ctypes.c_void_p()
        _call("ttrt_hook_output", self._h, ctypes.byref(h))
        return Tensor(h) if h.value else None

    __call__ = output

    def loc(self):
        buf = ctypes.create_string_buffer(512)
        _call("ttrt_hook_loc", self._h, buf, 512)
        return buf.value.decode("utf-8", "replace")

    def _refs(self, fn):
        ids, n = (ctypes.c_uint32 * 64)(), ctypes.c_uint32()
        _call(fn, self._h, ids, 64, ctypes.byref(n))
        return list(ids[: n.value])

    def input_refs(self):
        """global ids of the op's tensor operands (getOpInputRefs)."""
        return self._refs("ttrt_hook_input_refs")

    def output_refs(self):
        return self._refs("ttrt_hook_output_refs")

    def retrieve(self, global_id, untilize=True):
        """Host copy of a live tensor of the running program, or None (retrieveTensorFromPool)."""
        h = ctypes.c_void_p()
        _call("ttrt_hook_retrieve", self._h, global_id, int(untilize), ctypes.byref(h))
        return Tensor(h) if h.value else None

    def update(self, global_id, tensor):
        """Overwrite the payload of a pool tensor; `tensor` is converted to the pool tensor's layout (updateTensorInPool)."""
        _call("ttrt_hook_update", self._h, global_id, tensor.h)

    def program_index(self):
        i = ctypes.c_uint32()
        _call("ttrt_hook_program_index", self._h, ctypes.byref(i))
        return i.value

    def invoke_cpu_op(self, inputs):
        """Run the function behind the CpuOp this hook is at on host Tensors `inputs`; the list of its outputs (invokeCpuOp)."""
        arr = (ctypes.c_void_p * max(1, len(inputs)))(*[t.h for t in inputs])
        outs, n = (ctypes.c_void_p * 16)(), ctypes.c_uint32()
        _call("ttrt_hook_invoke_cpu_op", self._h, arr, len(inputs), outs, 16, ctypes.byref(n))
        return [Tensor(ctypes.c_void_p(outs[i])) for i in range(n.value)]

    def ref_desc(self, global_id):
        """(shape, dtype) of one of the op's operands or results as the binary declares it (TensorRef.get_shape / get_dtype)."""
        shape, rank, dt = (ctypes.c_uint32 * 8)(), ctypes.c_int(), ctypes.c_int()
        _call("ttrt_hook_ref_desc", self._h, global_id, shape, ctypes.byref(rank), ctypes.byref(dt))
        return list(shape[: rank.value]), dt.value


# An exception cannot cross the C frames between a callback and submit(): the first one a callback raises is kept, the
# callbacks after it do nothing, and submit() raises it when the program returns (the reference's bindings let it travel
# through, runtime/test/ttnn/python/n150/test_debug_hooks.py:416-458: the caller sees the callback's exception either way).
_callback_error = []


def _guarded(fn, *args):
    if _callback_error:
        return
    try:
        fn(*args)
    except BaseException as e:
        _callback_error.append(e)


def _raise_callback_error():
    if _callback_error:
        e = _callback_error[0]
        del _callback_error[:]
        raise e


def _op_trampoline(fn):
    def tramp(idx, name, dbg, hook, user):
        _guarded(fn, idx, name.decode("utf-8", "replace"), dbg.decode("utf-8", "replace"), HookContext(hook))
    return _CB_TYPE(tramp)


def set_post_op_callback(fn):
    """fn(op_index, op_name, debug_info, hook: HookContext), after every operation."""
    _cb_keep["post_op"] = _op_trampoline(fn)
    _call("ttrt_set_post_op_callback", _cb_keep["post_op"], None)


def set_pre_op_callback(fn):
    """fn(op_index, op_name, debug_info, hook: HookContext), before every operation."""
    _cb_keep["pre_op"] = _op_trampoline(fn)
    _call("ttrt_set_pre_op_callback", _cb_keep["pre_op"], None)


def set_program_callbacks(pre=None, post=None):
    """pre / post: fn(program_index, hook: HookContext) around every program, nested ones included."""
    def wrap(fn):
        if fn is None:
            return _PROGRAM_CB_TYPE()
        return _PROGRAM_CB_TYPE(lambda idx, hook, user: _guarded(fn, idx, HookContext(hook)))
    new_pre, new_post = wrap(pre), wrap(post)
    _call("ttrt_set_program_callbacks", new_pre, new_post, None)
    # a callback that is not given stays registered (the reference merges registrations,
    # runtime/test/ttnn/python/n150/test_debug_hooks.py:349-412): its trampoline must stay alive with it
    if pre is not None:
        _cb_keep["pre_program"] = new_pre
    if post is not None:
        _cb_keep["post_program"] = new_post


def walk_program(binary, program_index, fn):
    """fn(op_index, op_name, debug_info, hook: HookContext) for every operation of the program in order; nothing runs
    (walkProgram).  The hook answers loc / input_refs / output_refs / ref_desc; there is no tensor pool behind it."""
    raised = []

    def guarded(idx, name, dbg, hook):   # an exception cannot cross the C frames: keep the first, re-raise it afterwards
        if not raised:
            try:
                fn(idx, name, dbg, hook)
            except BaseException as e:
                raised.append(e)
    _call("ttrt_walk_program", binary.h, program_index, _op_trampoline(guarded), None)
    if raised:
        raise raised[0]


def clear_callbacks():
    _call("ttrt_clear_callbacks")
    _cb_keep.clear()


class ProgramBuilder:
    """Writes `.ttnn` programs; ids are flatbuffer global_ids (0 = no tensor)."""

    def __init__(self):
        self.h = ctypes.c_void_p()
        _call("ttrt_pb_create", ctypes.byref(self.h))

    def __del__(self):
        try:
            lib().ttrt_pb_destroy(self.h)
        except Exception:
            pass

    def begin_program(self, name, private=False):
        _call("ttrt_pb_begin_program", self.h, name.encode(), int(private))

    def end_program(self):
        i = ctypes.c_uint32()
        _call("ttrt_pb_end_program", self.h, ctypes.byref(i))
        return i.value

    def input(self, shape, dtype, layout=TensorLayout.Tile, storage=StorageType.Device):
        s, r = _shape_arg(shape)
        out = ctypes.c_uint32()
        _call("ttrt_pb_input", self.h, s, r, ctypes.byref(Layout(storage, layout, dtype)), ctypes.byref(out))
        return out.value

    def output(self, t):
        _call("ttrt_pb_output", self.h, t)

    def finish(self):
        data, size = ctypes.POINTER(ctypes.c_uint8)(), ctypes.c_size_t()
        _call("ttrt_pb_finish", self.h, ctypes.byref(data), ctypes.byref(size))
        out = ctypes.string_at(data, size.value)
        lib().ttrt_free_bytes(data)
        return out

    def desc(self, t):
        shape, rank, lay = (ctypes.c_uint32 * 8)(), ctypes.c_int(), Layout()
        _call("ttrt_pb_tensor_desc", self.h, t, shape, ctypes.byref(rank), ctypes.byref(lay))
        return tuple(shape[: rank.value]), lay

    def declare_next_shape(self, shape):
        """The next tensor the builder creates is declared with `shape` instead of the one its operation gives (a program that
        lies about a result, for tests of the executor's checks)."""
        sh, rank = _shape_arg(shape)
        _call("ttrt_pb_declare_next_shape", self.h, sh, rank)

    def last_op_loc(self):
        buf = ctypes.create_string_buffer(512)
        _call("ttrt_pb_last_op_loc", self.h, buf, 512)
        return buf.value.decode("utf-8", "replace")

    def golden(self, loc, array, dtype, name=""):
        """Embed an expected tensor for the op at `loc`: numpy array (bf16 as uint16 bits) of runtime dtype `dtype`."""
        import numpy as np
        a = np.ascontiguousarray(array)
        shape = (ctypes.c_int64 * max(1, a.ndim))(*a.shape)
        _call("ttrt_pb_golden", self.h, loc.encode(), name.encode(), a.ctypes.data_as(ctypes.c_void_p), a.nbytes, shape, a.ndim, dtype)

    def _op(self, name, *args):
        out = ctypes.c_uint32()
        _call(name, self.h, *args, ctypes.byref(out))
        return out.value

    def to_layout(self, t, layout, dtype=None, storage=StorageType.Device):
        return self._op("ttrt_pb_to_layout", t, layout, -1 if dtype is None else dtype, storage)

    def typecast(self, t, dtype):
        return self._op("ttrt_pb_typecast", t, dtype)

    def to_device(self, t):
        return self._op("ttrt_pb_to_device", t)

    def from_device(self, t):
        return self._op("ttrt_pb_from_device", t)

    def set_matmul_program_config(self, kind, fused_activation=-1):
        """The next matmul / linear carries a program config of this kind (1-4, the MatmulProgramConfig union) whose
        fused_activation is the given UnaryOpType (absent when negative)."""
        _call("ttrt_pb_set_matmul_program_config", self.h, int(kind), int(fused_activation))

    def matmul(self, a, b, transpose_a=False, transpose_b=False, activation="", out_dtype=DataType.BFloat16):
        return self._op("ttrt_pb_matmul", a, b, int(transpose_a), int(transpose_b), activation.encode(), out_dtype)

    def linear(self, a, b, bias=0, transpose_a=False, transpose_b=False, activation="", out_dtype=DataType.BFloat16):
        return self._op("ttrt_pb_linear", a, b, bias, int(transpose_a), int(transpose_b), activation.encode(), out_dtype)

    def unary(self, type_, t, param=None):
        return self._op("ttrt_pb_unary", type_, t, int(param is not None), ctypes.c_float(param or 0.0))

    def binary(self, type_, a, b):
        return self._op("ttrt_pb_binary", type_, a, b)

    def rms_norm(self, t, weight=0, bias=0, eps=1e-5):
        return self._op("ttrt_pb_rms_norm", t, weight, bias, ctypes.c_float(eps))

    def softmax(self, t, dim=-1):
        return self._op("ttrt_pb_softmax", t, dim)

    def reduction(self, type_, t, dims, keep_dim=False):
        d = (ctypes.c_int32 * max(1, len(dims)))(*dims)
        return self._op("ttrt_pb_reduction", type_, t, d, len(dims), int(keep_dim))

    def sdpa(self, q, k, v, mask=0, is_causal=False, scale=None, sliding_window=None, attention_sink=0):
        return self._op("ttrt_pb_sdpa", q, k, v, mask, int(is_causal), int(scale is not None), ctypes.c_float(scale or 0.0),
                        ctypes.c_int64(-1 if sliding_window is None else sliding_window), attention_sink)

    def rotary_embedding(self, t, cos_cache, sin_cache, token_index=None):
        return self._op("ttrt_pb_rotary_embedding", t, cos_cache, sin_cache, int(token_index is not None), token_index or 0)

    def update_cache(self, cache, t, update_index, batch_offset=0):
        _call("ttrt_pb_update_cache", self.h, cache, t, update_index, batch_offset)

    def fill_cache(self, cache, t, batch_offset=0):
        _call("ttrt_pb_fill_cache", self.h, cache, t, batch_offset)

    def paged_update_cache(self, cache, t, update_index, page_table=0, share_cache=False):
        _call("ttrt_pb_paged_update_cache", self.h, cache, t, update_index, page_table, int(share_cache))

    def paged_fill_cache(self, cache, t, page_table, batch_idx=0):
        _call("ttrt_pb_paged_fill_cache", self.h, cache, t, page_table, batch_idx)

    def sdpa_decode(self, q, k, v, cur_pos=0, mask=0, page_table=0, is_causal=True, scale=None, sliding_window=None,
                    attention_sink=0):
        return self._op("ttrt_pb_sdpa_decode", q, k, v, page_table, mask, cur_pos, int(is_causal), int(scale is not None),
                        ctypes.c_float(scale or 0.0), ctypes.c_int64(-1 if sliding_window is None else sliding_window), attention_sink)

    def reshape(self, t, shape):
        s, r = _shape_arg(shape)
        return self._op("ttrt_pb_reshape", t, s, r)

    def permute(self, t, perm):
        p = (ctypes.c_int64 * len(perm))(*perm)
        return self._op("ttrt_pb_permute", t, p, len(perm))

    def transpose(self, t, dim0, dim1):
        return self._op("ttrt_pb_transpose", t, dim0, dim1)

    def concat(self, ts, dim):
        a = (ctypes.c_uint32 * len(ts))(*ts)
        return self._op("ttrt_pb_concat", a, len(ts), dim)

    def slice(self, t, begins, ends, steps=None):
        n = len(begins)
        steps = steps or [1] * n
        mk = lambda v: (ctypes.c_int64 * n)(*v)
        return self._op("ttrt_pb_slice", t, mk(begins), mk(ends), mk(steps), n)

    def repeat_interleave(self, t, repeats, dim):
        return self._op("ttrt_pb_repeat_interleave", t, repeats, dim)

    def unary_composite(self, type_, t, lo=0.0, hi=0.0, int_bounds=False):
        return self._op("ttrt_pb_unary_composite", type_, t, ctypes.c_float(lo), ctypes.c_float(hi), int(int_bounds))

    def concatenate_heads(self, t):
        return self._op("ttrt_pb_concat_heads", 0, t, 0)

    def nlp_concat_heads(self, t):
        return self._op("ttrt_pb_concat_heads", 1, t, 0)

    def nlp_concat_heads_decode(self, t, num_heads):
        return self._op("ttrt_pb_concat_heads", 2, t, num_heads)

    def nlp_create_qkv_heads_decode(self, t, num_heads, num_kv_heads):
        out = (ctypes.c_uint32 * 3)()
        _call("ttrt_pb_nlp_create_qkv_heads_decode", self.h, t, num_heads, num_kv_heads, out)
        return tuple(out)

    def split_query_key_value_and_split_heads(self, t, num_heads, num_kv_heads=None, kv_input=0, transpose_key=False):
        out = (ctypes.c_uint32 * 3)()
        _call("ttrt_pb_split_qkv_and_split_heads", self.h, t, kv_input, num_heads, num_kv_heads or num_heads, int(transpose_key), out)
        return tuple(out)

    def repeat(self, t, repeats):
        r = (ctypes.c_int64 * len(repeats))(*repeats)
        return self._op("ttrt_pb_repeat", t, r, len(repeats))

    def binary_composite(self, type_, lhs, rhs):
        return self._op("ttrt_pb_binary_composite", type_, lhs, rhs)

    def where(self, cond, a, b):
        return self._op("ttrt_pb_where", cond, a, b)

    def embedding(self, indices, weight):
        return self._op("ttrt_pb_embedding", indices, weight)

    def argmax(self, t, dim=None, keep_dim=False, out_dtype=None):
        return self._op("ttrt_pb_argmax", t, int(dim is not None), dim or 0, int(keep_dim),
                        int(DataType.Int32 if out_dtype is None else out_dtype))

    def arange(self, start, end, step=1, dtype=None, layout=None):
        return self._op("ttrt_pb_arange", ctypes.c_float(start), ctypes.c_float(end), ctypes.c_float(step),
                        int(DataType.Float32 if dtype is None else dtype), int(TensorLayout.RowMajor if layout is None else layout))

    def constant(self, array, in_dtype, dtype=None, layout=TensorLayout.Tile, storage=StorageType.Device):
        a = np.ascontiguousarray(array)
        s, r = _shape_arg(a.shape)
        lay = Layout(storage, layout, in_dtype if dtype is None else dtype)
        return self._op("ttrt_pb_constant", ctypes.c_void_p(a.ctypes.data), ctypes.c_size_t(a.nbytes), in_dtype, s, r, ctypes.byref(lay))

    def full(self, shape, value, dtype, layout=TensorLayout.Tile):
        s, r = _shape_arg(shape)
        return self._op("ttrt_pb_full", s, r, ctypes.c_float(value), dtype, layout)

    def empty(self, shape, dtype, layout=TensorLayout.Tile):
        s, r = _shape_arg(shape)
        return self._op("ttrt_pb_empty", s, r, dtype, layout)

    def copy(self, src, dst):
        _call("ttrt_pb_copy", self.h, src, dst)

    def write_tensor(self, host, device):
        _call("ttrt_pb_write_tensor", self.h, host, device)

    def begin_trace_capture(self):
        return self._op("ttrt_pb_begin_trace_capture")

    def end_trace_capture(self, trace_id):
        _call("ttrt_pb_end_trace_capture", self.h, trace_id)

    def execute_trace(self, trace_id, blocking=False):
        _call("ttrt_pb_execute_trace", self.h, trace_id, int(blocking))

    def capture_or_execute_trace(self, capture_program, execute_program, allocate_slots_program, ins, out_descs):
        return self._multi("ttrt_pb_capture_or_execute_trace", (capture_program, execute_program, allocate_slots_program), ins, out_descs)

    def deallocate(self, t, force=False):
        _call("ttrt_pb_deallocate", self.h, t, int(force))

    def _multi(self, name, head, ins, out_descs):
        n_out = len(out_descs)
        shapes = (ctypes.c_uint32 * (8 * n_out))()
        ranks = (ctypes.c_int * n_out)()
        lays = (Layout * n_out)()
        for i, (shape, lay) in enumerate(out_descs):
            for j, s in enumerate(shape):
                shapes[8 * i + j] = s
            ranks[i] = len(shape)
            lays[i] = lay
        ia = (ctypes.c_uint32 * max(1, len(ins)))(*ins)
        outs = (ctypes.c_uint32 * n_out)()
        _call(name, self.h, *head, ia, len(ins), shapes, ranks, lays, n_out, outs)
        return list(outs)

    def load_cached(self, program_index, callee, ins, out_descs):
        return self._multi("ttrt_pb_load_cached", (program_index, callee.encode()), ins, out_descs)

    def func_call(self, program_index, ins, out_descs):
        return self._multi("ttrt_pb_func_call", (program_index,), ins, out_descs)

    def rotary_embedding_llama(self, t, cos_cache, sin_cache, trans_mat, decode_mode=False):
        return self._op("ttrt_pb_rotary_embedding_llama", t, cos_cache, sin_cache, trans_mat, int(decode_mode))

    def chunked_sdpa(self, q, k, v, page_table, chunk_start, scale=None):
        return self._op("ttrt_pb_chunked_sdpa", q, k, v, page_table, chunk_start, int(scale is not None), ctypes.c_float(scale or 0.0))

    def add_dylib(self, dylib_id, data):
        """Embed a shared library (bytes) in the open program; cpu_op calls functions of it."""
        buf = (ctypes.c_uint8 * len(data)).from_buffer_copy(data)
        _call("ttrt_pb_add_dylib", self.h, dylib_id, buf, len(data))

    def cpu_op(self, dylib_id, func_name, ins, out_descs):
        return self._multi("ttrt_pb_cpu_op", (dylib_id, func_name.encode()), ins, out_descs)
