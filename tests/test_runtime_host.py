"""Host-side runtime logic that needs no GPU: the flatbuffer codec, binary inspection, host tensor
creation (strides, unsupported dtype aliases) and the buffer casts with the reference's
known-answer vectors."""
import ctypes
import os
import struct

import numpy as np
import pytest

from ttmlir_amd import runtime as rt, programs

DT, TL, ST = rt.DataType, rt.TensorLayout, rt.StorageType


def test_runtime_abi_symbols():
    l = ctypes.CDLL(rt.LIB_PATH)
    names = rt.declared_functions()
    assert len(names) > 60
    for n in names:
        assert hasattr(l, n), "declared but not exported: " + n


def test_binary_wire_format_and_inspection(tmp_path):
    data = programs.c1_matmul()
    # size-prefixed flatbuffer with file identifier "TTNN" (include/ttmlir/Target/TTNN/binary.fbs:17-19)
    assert struct.unpack("<I", data[:4])[0] == len(data) - 4
    assert data[8:12] == b"TTNN"
    root = struct.unpack("<I", data[4:8])[0]
    assert 0 < root < len(data) - 4 and root % 4 == 0
    b = rt.Binary.load_from_memory(data)
    assert b.info() == ("TTNN", "0.1.0")
    assert b.get_num_programs() == 1 and b.get_program_name(0) == "c1_matmul"
    ins, outs = b.get_program_inputs(0), b.get_program_outputs(0)
    assert [s for s, _ in ins] == [(256, 512), (512, 256)]
    assert all(l == rt.Layout(ST.Host, TL.RowMajor, DT.BFloat16) for _, l in ins)
    assert outs[0] == ((256, 256), rt.Layout(ST.Host, TL.RowMajor, DT.BFloat16))
    assert outs[1] == ((256, 512), rt.Layout(ST.Device, TL.Tile, DT.BFloat16))
    text = b.get_program_ops_as_text(0)
    assert [l.split()[1] for l in text.strip().splitlines()] == ["ToDeviceOp", "ToLayoutOp", "ToDeviceOp", "ToLayoutOp", "MatmulOp",
                                                                "ToLayoutOp", "FromDeviceOp"]
    p = tmp_path / "c1.ttnn"
    b.store(p)
    assert rt.Binary.load_from_path(p).get_program_name(0) == "c1_matmul"
    assert rt.get_layout(b, 0, 1) == rt.Layout(ST.Host, TL.RowMajor, DT.BFloat16)


def test_const_eval_program_structure():
    b = rt.Binary.load_from_memory(programs.c4_mlp(tokens=64, hidden=128, ffn=256))
    assert b.get_num_programs() == 2
    assert b.is_program_private(0) and not b.is_program_private(1)
    assert [l.dtype for _, l in b.get_program_outputs(0)] == [DT.BFP_BFloat8, DT.BFP_BFloat8, DT.BFP_BFloat4]
    ops = [l.split()[1] for l in b.get_program_ops_as_text(1).strip().splitlines()]
    assert ops == ["LoadCachedOp", "RMSNormOp", "LinearOp", "MatmulOp", "EltwiseBinaryOp", "DeallocateOp", "DeallocateOp", "MatmulOp",
                   "DeallocateOp"]


def test_json_views_of_a_program():
    b = rt.Binary.load_from_memory(programs.c4_mlp(tokens=64, hidden=128, ffn=256))
    ins = b.get_program_inputs_as_json(1)
    assert [t["desc"]["shape"] for t in ins] == [[64, 128], [128], [128, 256], [128, 256], [256, 128]]
    md = ins[0]["desc"]["layout"]["memory_desc"]
    assert md["data_type"] == "BFloat16" and md["tile_shape"] == {"y": 32, "x": 32} and md["storage_type"] == "DRAM"
    assert len({t["global_id"] for t in ins}) == 5
    outs = b.get_program_outputs_as_json(1)
    assert [t["desc"]["shape"] for t in outs] == [[64, 128]]
    assert [t["desc"]["layout"]["memory_desc"]["data_type"] for t in b.get_program_outputs_as_json(0)] == [
        "BFP_BFloat8", "BFP_BFloat8", "BFP_BFloat4"]
    ops = b.get_program_ops_as_json(1)
    text = b.get_program_ops_as_text(1).strip().splitlines()
    assert [o["type_type"] for o in ops] == [l.split()[1] for l in text]
    assert all(set(o) == {"type_type", "debug_info", "loc_info"} for o in ops)
    assert [o["loc_info"] for o in ops] == ['loc("c4_mlp"("op%d"))' % i for i in range(len(ops))]
    with pytest.raises(RuntimeError, match="out of range"):
        b.get_program_ops_as_json(5)


def test_embedded_goldens_round_trip():
    """DebugInfo.golden_info (include/ttmlir/Target/Common/debug_info.fbs:6-26) written by the builder and read back."""
    pb = rt.ProgramBuilder()
    pb.begin_program("g")
    a, w = pb.input((32, 64), DT.BFloat16), pb.input((64, 32), DT.BFloat16)
    c = pb.matmul(a, w)
    loc_mm = pb.last_op_loc()
    r = pb.unary(programs.UNARY["relu"], c)
    loc_relu = pb.last_op_loc()
    assert (loc_mm, loc_relu) == ('loc("g"("op0"))', 'loc("g"("op1"))')
    want = np.linspace(-4, 4, 32 * 32, dtype=np.float32).reshape(32, 32)
    bits = (want.view(np.uint32) >> 16).astype(np.uint16)
    pb.golden(loc_mm, bits, DT.BFloat16, "product")
    pb.golden(loc_relu, np.array([[1.5, -2.25, 3.0]], dtype=np.float32), DT.Float32, "relu")
    pb.golden("input_0", np.arange(6, dtype=np.int32).reshape(1, 2, 3), DT.Int32)
    pb.output(r)
    pb.end_program()
    b = rt.Binary.load_from_memory(pb.finish())
    name, got = b.get_debug_info_golden(loc_mm)
    assert name == "product" and got.dtype == np.float32 and got.shape == (32, 32)
    assert np.array_equal(got.view(np.uint32), bits.astype(np.uint32) << 16)
    name, got = b.get_debug_info_golden(loc_relu)
    assert name == "relu" and np.array_equal(got, np.array([[1.5, -2.25, 3.0]], dtype=np.float32))
    name, got = b.get_debug_info_golden("input_0")
    assert name == "" and got.dtype == np.int32 and np.array_equal(got, np.arange(6).reshape(1, 2, 3))
    assert b.get_debug_info_golden('loc("g"("op7"))') is None
    # binaries without debug info answer "no golden" rather than failing
    assert rt.Binary.load_from_memory(programs.c1_matmul()).get_debug_info_golden(loc_mm) is None
    # golden with a byte count that does not match shape x dtype is refused when it is recorded
    with pytest.raises(RuntimeError, match="golden"):
        pb2 = rt.ProgramBuilder()
        pb2.begin_program("h")
        pb2.golden("x", np.zeros(5, dtype=np.uint8), DT.Float32)


def test_program_goldens_option_marks_each_stage():
    st = {k: np.full(s, i + 1, dtype=np.float32) for i, (k, s) in enumerate(
        dict(norm=(64, 128), gate=(64, 256), up=(64, 256), product=(64, 256), down=(64, 128)).items())}
    b = rt.Binary.load_from_memory(programs.c4_mlp(64, 128, 256, goldens=st))
    ops = b.get_program_ops_as_json(1)
    found = {}
    for o in ops:
        g = b.get_debug_info_golden(o["loc_info"])
        if g is not None:
            found[g[0]] = (o["type_type"], g[1])
    assert {k: v[0] for k, v in found.items()} == dict(norm="RMSNormOp", gate="LinearOp", up="MatmulOp", product="EltwiseBinaryOp",
                                                        down="MatmulOp")
    assert all(np.array_equal(found[k][1], st[k]) for k in st)


def test_ttrt_read_and_error_records(tmp_path, capsys):
    import json
    from ttmlir_amd import ttrt
    path = tmp_path / "c4.ttnn"
    path.write_bytes(programs.c4_mlp(64, 128, 256, goldens={"norm": np.ones((64, 128), np.float32),
                                                              "output_0": np.zeros((64, 128), np.float32)}))
    assert ttrt.main(["read", str(path)]) == 0
    info = json.loads(capsys.readouterr().out)
    assert info["file_identifier"] == "TTNN" and [p["private"] for p in info["programs"]] == [True, False]
    assert [o["type_type"] for o in info["ops"][1]][:2] == ["LoadCachedOp", "RMSNormOp"]
    assert info["goldens"][0] == []
    assert [(g["loc"], g["name"], g["shape"]) for g in info["goldens"][1]] == [
        ('loc("c4_mlp"("op1"))', "norm", [64, 128]), ("output_0", "output_0", [64, 128])]
    assert ttrt.main(["read", str(path), "--section", "version"]) == 0
    assert set(json.loads(capsys.readouterr().out)) == {"file_path", "file_identifier", "version"}
    # a binary that cannot be read becomes an error record and a non-zero exit code, not a traceback
    res = tmp_path / "r.json"
    assert ttrt.main(["run", str(tmp_path / "missing.ttnn"), "--result-file", str(res)]) == 1
    (rec,) = json.loads(res.read_text())
    assert rec["result"] == "error" and "cannot open" in rec["exception"] and rec["program_results"] == []


def test_ttrt_input_initialisers():
    import torch
    from ttmlir_amd import ttrt
    g = torch.Generator().manual_seed(0)
    a = ttrt.make_input((4, 8), DT.BFloat16, "randn", g)
    want = torch.randn((4, 8), generator=torch.Generator().manual_seed(0)).to(torch.bfloat16)
    assert a.dtype == torch.bfloat16 and torch.equal(a, want)
    assert torch.equal(ttrt.make_input((2, 3), DT.Float32, "arange", g), torch.arange(6.0).reshape(2, 3))
    idx = ttrt.make_input((16,), DT.Int32, "randn", g)
    assert idx.dtype == torch.int32 and int(idx.min()) >= 0 and int(idx.max()) < 8
    assert ttrt.make_input((2, 2), DT.BFP_BFloat8, "ones", g).dtype == torch.bfloat16


def test_decoder_program_shapes():
    b = rt.Binary.load_from_memory(programs.c5_decoder(seq=64, hidden=256, n_q=4, n_kv=2, head_dim=64, ffn=512))
    assert b.get_program_outputs(1)[0][0] == (1, 64, 256)
    assert len(b.get_program_inputs(1)) == 10
    assert "ScaledDotProductAttentionOp" in b.get_program_ops_as_text(1)


@pytest.mark.parametrize("bad", [b"", b"\x00" * 8, b"\x10\x00\x00\x00" + b"\x00" * 16, b"garbage-that-is-not-a-flatbuffer!"])
def test_malformed_binaries_are_rejected(bad):
    with pytest.raises(RuntimeError):
        rt.Binary.load_from_memory(bad)


def test_truncated_binary_is_rejected():
    data = programs.c1_matmul()
    with pytest.raises(RuntimeError):
        rt.Binary.load_from_memory(data[: len(data) // 2])
    wrong = bytearray(data)
    wrong[8:12] = b"TTM0"
    with pytest.raises(RuntimeError):
        rt.Binary.load_from_memory(bytes(wrong))


def test_buffer_cast_known_answers():
    # runtime/test/common/gtest/test_handle_float_bfloat_buffer_cast.cpp:8-46
    f16 = np.array([0xBC00, 0, 0xBC00], dtype=np.uint16).view(np.float16)
    assert rt.buffer_cast(f16, DT.Float16, DT.BFloat16).tolist() == [0xBF80, 0, 0xBF80]
    bf = np.array([0xBF80, 0, 0xBF80], dtype=np.uint16)
    assert rt.buffer_cast(bf, DT.BFloat16, DT.Float16).view(np.uint16).tolist() == [0xBC00, 0, 0xBC00]
    mm = np.array([0xFBFF, 0x7BFF], dtype=np.uint16).view(np.float16)
    assert rt.buffer_cast(mm, DT.Float16, DT.BFloat16).tolist() == [0xC780, 0x4780]


def test_integer_buffer_casts_saturate():
    # runtime/test/common/gtest/test_handle_integer_buffer_cast.cpp:8-66: clamp to the destination range
    i64 = np.array([0, -1, 2 ** 31 - 1, 2 ** 31, -2 ** 31 - 1, 2 ** 62, -2 ** 62], dtype=np.int64)
    assert rt.buffer_cast(i64, DT.Int64, DT.Int32).tolist() == [0, -1, 2 ** 31 - 1, 2 ** 31 - 1, -2 ** 31, 2 ** 31 - 1, -2 ** 31]
    u64 = np.array([0, 2 ** 32 - 1, 2 ** 32, 2 ** 63], dtype=np.uint64)
    assert rt.buffer_cast(u64, DT.UInt64, DT.UInt32).tolist() == [0, 2 ** 32 - 1, 2 ** 32 - 1, 2 ** 32 - 1]
    i16 = np.array([-5, 0, 7, -32768, 32767], dtype=np.int16)
    assert rt.buffer_cast(i16, DT.Int16, DT.UInt16).tolist() == [0, 0, 7, 0, 32767]
    u16 = np.array([0, 32767, 32768, 65535], dtype=np.uint16)
    assert rt.buffer_cast(u16, DT.UInt16, DT.Int16).tolist() == [0, 32767, 32767, 32767]
    i8 = np.array([-128, -1, 0, 127], dtype=np.int8)
    assert rt.buffer_cast(i8, DT.Int8, DT.UInt8).tolist() == [0, 0, 0, 127]
    assert rt.buffer_cast(np.array([1, 2 ** 31 - 1], dtype=np.int32), DT.Int32, DT.Int64).tolist() == [1, 2 ** 31 - 1]
    assert rt.buffer_cast(np.array([2 ** 32 - 1], dtype=np.uint32), DT.UInt32, DT.Int64).tolist() == [2 ** 32 - 1]
    f64 = np.array([1.5, -2.25, 1e300], dtype=np.float64)
    assert rt.buffer_cast(f64, DT.Float64, DT.Float32).tolist() == [1.5, -2.25, float("inf")]
    with pytest.raises(RuntimeError):
        rt.buffer_cast(f64, DT.Float64, DT.Int32)


def test_owned_host_tensor_gathers_strides():
    # runtime/test/ttnn/gtest/test_owned_host_tensor_strided.cpp:44-92: element strides, non-contiguous source
    base = np.arange(24, dtype=np.float32).reshape(4, 6)
    t = rt.create_owned_host_tensor(base, DT.Float32, stride=None)
    assert np.array_equal(rt.to_numpy(t), base)
    # view of every other column: shape [4,3], strides (6, 2) elements
    src = np.ascontiguousarray(base)
    h = ctypes.c_void_p()
    shape = (ctypes.c_uint32 * 8)(4, 3)
    stride = (ctypes.c_int64 * 8)(6, 2)
    assert rt.lib().ttrt_tensor_create_host(ctypes.c_void_p(src.ctypes.data), shape, 2, stride, 4, DT.Float32, 0, ctypes.byref(h)) == 0
    assert np.array_equal(rt.to_numpy(rt.Tensor(h)), base[:, ::2])
    # a transposed view
    stride = (ctypes.c_int64 * 8)(1, 6)
    shape = (ctypes.c_uint32 * 8)(6, 4)
    assert rt.lib().ttrt_tensor_create_host(ctypes.c_void_p(src.ctypes.data), shape, 2, stride, 4, DT.Float32, 0, ctypes.byref(h)) == 0
    assert np.array_equal(rt.to_numpy(rt.Tensor(h)), base.T)
    # borrowed tensors must be contiguous
    assert rt.lib().ttrt_tensor_create_host(ctypes.c_void_p(src.ctypes.data), shape, 2, stride, 4, DT.Float32, 1, ctypes.byref(h)) == 1
    assert b"non-contiguous" in rt.lib().ttrt_last_error()


def test_unsupported_host_dtypes_are_aliased():
    # i64 -> i32 with saturation on the way in, cast back on the way out (runtime/lib/ttnn/runtime.cpp:120-141, 999-1041)
    x = np.array([[1, -2, 2 ** 40], [3, 4, -2 ** 40]], dtype=np.int64)
    t = rt.create_owned_host_tensor(x, DT.Int64)
    assert t.layout.dtype == DT.Int32
    back = rt.to_numpy(t, target_dtype=DT.Int64)
    assert back.dtype == np.int64 and back.tolist() == [[1, -2, 2 ** 31 - 1], [3, 4, -2 ** 31]]
    f = rt.create_owned_host_tensor(np.array([1.5, 2.5], dtype=np.float64), DT.Float64)
    assert f.layout.dtype == DT.Float32 and rt.to_numpy(f).tolist() == [1.5, 2.5]
    b = rt.create_owned_host_tensor(np.array([True, False, True]), DT.Bool)
    assert b.layout.dtype == DT.BFloat16 and rt.to_numpy(b).tolist() == [0x3F80, 0, 0x3F80]
    h = rt.create_owned_host_tensor(np.array([1.0, -2.0], dtype=np.float16), DT.Float16)
    assert h.layout.dtype == DT.BFloat16 and rt.to_numpy(h).tolist() == [0x3F80, 0xC000]


def test_borrowed_tensor_aliases_and_retain_flag():
    a = np.arange(6, dtype=np.float32).reshape(2, 3)
    t = rt.create_borrowed_host_tensor(a, DT.Float32)
    a[0, 0] = 42.0
    assert rt.to_numpy(t)[0, 0] == 42.0
    assert not t.get_retain()
    t.set_retain(True)
    assert t.get_retain()
    with pytest.raises(RuntimeError):
        rt.create_owned_host_tensor(np.zeros(4, np.uint8), DT.BFP_BFloat8)


def test_submit_without_device_fails_cleanly():
    if rt.get_num_available_devices() > 0:
        pytest.skip("a GPU is visible")
    with pytest.raises(RuntimeError):
        rt.open_mesh_device()


def test_schema_constants_are_what_the_generator_makes_of_the_schema_text():
    """schema_generated.h / schema_names.cpp say "generated": the generator sits beside them and reproduces them from the
    .fbs files of the tt-mlir checkout, where one is at hand (it is not on the GPU box)."""
    import importlib.util
    ref = "/root/reference"
    if not os.path.isdir(os.path.join(ref, "include", "ttmlir", "Target", "TTNN")):
        pytest.skip("no tt-mlir checkout at " + ref)
    rtdir = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "tt-mlir_amd", "runtime")
    spec = importlib.util.spec_from_file_location("gen_schema", os.path.join(rtdir, "gen_schema.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    for fname, text in gen.generate(ref).items():
        assert open(os.path.join(rtdir, fname)).read() == text, fname + " differs from the generator's output"


def _program_with_recorded_descs():
    """A two-program binary written with the program builder, and per program the (op name, input descs, output descs)
    the builder reported while writing it: what the walk must find in the flatbuffer."""
    pb = rt.ProgramBuilder()
    want = []
    pb.begin_program("prep", private=True)
    w = pb.input((96, 40), DT.BFloat16)
    wq = pb.typecast(w, DT.BFP_BFloat8)
    pb.output(wq)
    pb.end_program()
    want.append([("TypecastOp", [w], [wq], pb)])
    pb.begin_program("main")
    x = pb.input((2, 33, 96), DT.BFloat16)
    g = pb.input((96,), DT.BFloat16)
    wi = pb.input((96, 40), DT.BFP_BFloat8)
    n = pb.rms_norm(x, g, eps=1e-5)
    y = pb.matmul(n, wi)
    s = pb.softmax(y, dim=-1)
    r = pb.reduction(0, s, [2], keep_dim=True)
    t = pb.transpose(y, 1, 2)
    pb.output(r)
    pb.output(t)
    pb.end_program()
    want.append([("RMSNormOp", [x, g], [n], pb), ("MatmulOp", [n, wi], [y], pb), ("SoftmaxOp", [y], [s], pb),
                 ("ReductionOp", [s], [r], pb), ("TransposeOp", [y], [t], pb)])
    descs = {i: pb.desc(i) for ops in want for _, ins, outs, _ in ops for i in ins + outs}
    return rt.Binary.load_from_memory(pb.finish()), [[(name, ins, outs) for name, ins, outs, _ in ops] for ops in want], descs


def test_walk_program_reports_every_operation_with_its_tensor_refs():
    # the reference's own check of walkProgram (test/python/chisel/test_walk_program.py:14-54): every operation in order,
    # the shapes of its operand and result references equal to the shapes of the program that was compiled
    binary, want, descs = _program_with_recorded_descs()
    for program, ops in enumerate(want):
        seen = []

        def visit(idx, name, dbg, hook):
            ins, outs = hook.input_refs(), hook.output_refs()
            seen.append((idx, name, ins, outs))
            for gid in ins + outs:
                shape, dtype = hook.ref_desc(gid)
                assert tuple(shape) == tuple(descs[gid][0]) and dtype == descs[gid][1].dtype
            assert hook.loc() == 'loc("%s"("op%d"))' % (binary.get_program_name(program), idx) and dbg.startswith("ttnn.")
            assert hook.output() is None and hook.retrieve(ins[0]) is None   # nothing runs: there is no tensor pool
            with pytest.raises(rt.RuntimeError_, match="no program context"):
                hook.program_index()
            with pytest.raises(rt.RuntimeError_, match="neither an operand nor a result"):
                hook.ref_desc(10 ** 6)
        rt.walk_program(binary, program, visit)
        assert [(n, i, o) for _, n, i, o in seen] == ops
        assert [i for i, _, _, _ in seen] == list(range(len(ops)))


def test_walk_program_errors():
    binary, _, _ = _program_with_recorded_descs()
    with pytest.raises(rt.RuntimeError_, match="program index out of range"):
        rt.walk_program(binary, 2, lambda *a: None)

    class Stop(Exception):
        pass
    calls = []

    def boom(idx, *a):
        calls.append(idx)
        raise Stop()
    with pytest.raises(Stop):
        rt.walk_program(binary, 1, boom)
    assert calls == [0]   # the first exception ends the walk for the caller


@pytest.mark.parametrize("dtype,np_dtype", [(DT.Float32, np.float32), (DT.BFloat16, np.uint16), (DT.Int32, np.int32), (DT.UInt8, np.uint8)])
def test_dump_and_load_tensor_round_trip(tmp_path, dtype, np_dtype):
    rng = np.random.default_rng(3)
    a = rng.integers(0, 200, size=(3, 5, 7)).astype(np_dtype)
    t = rt.create_owned_host_tensor(a, dtype)
    path = tmp_path / "t.tensor"
    rt.dump_tensor(t, path)
    back = rt.load_tensor(path)
    assert back.get_shape() == [3, 5, 7] and back.get_layout() == rt.Layout(ST.Host, TL.RowMajor, dtype)
    assert np.array_equal(rt.to_numpy(back), a)
    assert back.get_data_buffer() == bytearray(a.tobytes())
    # container: magic, version, dtype, layout, rank, extents, payload size, payload
    raw = path.read_bytes()
    assert raw[:4] == b"TTMT" and struct.unpack("<5I", raw[4:24]) == (1, dtype, TL.RowMajor, 3, 3)
    assert struct.unpack("<2I", raw[24:32]) == (5, 7) and struct.unpack("<Q", raw[32:40])[0] == a.nbytes
    assert raw[40:] == a.tobytes()


def test_load_tensor_rejects_damaged_files(tmp_path):
    a = np.arange(24, dtype=np.float32).reshape(4, 6)
    path = tmp_path / "t.tensor"
    rt.dump_tensor(rt.create_owned_host_tensor(a, DT.Float32), path)
    raw = path.read_bytes()

    def load(data):
        p = tmp_path / "bad.tensor"
        p.write_bytes(data)
        return rt.load_tensor(p)
    with pytest.raises(rt.RuntimeError_, match="not a tensor file"):
        load(b"XXXX" + raw[4:])
    with pytest.raises(rt.RuntimeError_, match="unknown tensor file version"):
        load(raw[:4] + struct.pack("<I", 9) + raw[8:])
    with pytest.raises(rt.RuntimeError_, match="ends inside its payload"):
        load(raw[:-8])
    with pytest.raises(rt.RuntimeError_, match="ends inside its header"):
        load(raw[:18])
    with pytest.raises(rt.RuntimeError_, match="payload size does not match"):
        load(raw[:28] + struct.pack("<I", 7) + raw[32:])           # second extent 6 -> 7
    with pytest.raises(rt.RuntimeError_, match="unknown data type"):
        load(raw[:8] + struct.pack("<I", 99) + raw[12:])
    with pytest.raises(rt.RuntimeError_, match="never stored in"):
        load(raw[:8] + struct.pack("<I", DT.Float64) + raw[12:])
    with pytest.raises(rt.RuntimeError_, match="block-float data outside the tile layout"):
        load(raw[:8] + struct.pack("<I", DT.BFP_BFloat8) + raw[12:])
    with pytest.raises(rt.RuntimeError_, match="cannot open"):
        rt.load_tensor(tmp_path / "absent.tensor")
    with pytest.raises(rt.RuntimeError_, match="cannot open"):
        rt.dump_tensor(rt.create_owned_host_tensor(a, DT.Float32), tmp_path / "no_such_dir" / "t.tensor")


def test_tensor_accessors_and_empty_host_tensors():
    a = np.zeros((2, 3, 40), dtype=np.float32)
    t = rt.create_owned_host_tensor(a, DT.Float32)
    assert t.get_shape() == [2, 3, 40] and t.get_stride() == [120, 40, 1]
    assert t.get_volume() == 240 and t.get_logical_volume() == 240 and t.get_element_size() == 4 and t.get_dtype() == DT.Float32
    assert t.has_layout(rt.Layout(ST.Host, TL.RowMajor, DT.Float32))
    assert not t.has_layout(rt.Layout(ST.Host, TL.Tile, DT.Float32))
    assert not t.has_layout(rt.Layout(ST.Device, TL.RowMajor, DT.Float32))
    assert not t.has_layout(rt.Layout(ST.Host, TL.RowMajor, DT.BFloat16))
    # host storage needs no device; the tile layout pads both trailing extents to 32, block-float tiles are 1088 / 576 bytes
    e = rt.create_empty_tensor(None, rt.Layout(ST.Host, TL.RowMajor, DT.BFloat16), (4, 10))
    assert e.is_allocated() and e.desc() == ((4, 10), rt.Layout(ST.Host, TL.RowMajor, DT.BFloat16), 80)
    e = rt.create_empty_tensor(None, rt.Layout(ST.Host, TL.Tile, DT.Float32), (2, 33, 40))
    assert e.desc()[2] == 2 * 64 * 64 * 4 and e.get_volume() == 2 * 64 * 64 and e.get_logical_volume() == 2 * 33 * 40
    e = rt.create_empty_tensor(None, rt.Layout(ST.Host, TL.Tile, DT.BFP_BFloat8), (33, 40))
    assert e.desc()[2] == 4 * 1088 and e.get_element_size() == 1
    e = rt.create_empty_tensor(None, rt.Layout(ST.Host, TL.Tile, DT.BFP_BFloat4), (64, 64))
    assert e.desc()[2] == 4 * 576
    with pytest.raises(rt.RuntimeError_, match="null argument: device"):
        rt.create_empty_tensor(None, rt.Layout(ST.Device, TL.Tile, DT.BFloat16), (32, 32))


def test_invoke_cpu_op_on_caller_inputs(tmp_path):
    """invokeCpuOp (runtime/lib/ttnn/runtime.cpp:2598-2611, runtime/lib/ttnn/operations/cpu/cpu.cpp:240-300): the function of a
    CpuOp on tensors the caller brings, checked against the op's declared inputs.  It needs the program's embedded library
    and nothing of a running program, so it is reachable from a walk of the binary (the reference's test of the call,
    runtime/test/ttnn/python/n150/test_cpu_hoisting_api.py:44-120, makes it from a post-op hook of a running program and
    checks the sum of two caller-supplied tensors, as here): the whole CpuOp path (library from the
    binary's bytes, WrappedTensor packing, ownership of what the callee allocated) runs here without a device."""
    import subprocess
    src = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "cpu_hoisted_ops.c")
    so = tmp_path / "hoisted.so"
    subprocess.run(["gcc", "-shared", "-fPIC", "-O1", "-o", str(so), src], check=True)
    host = lambda shape, dt: (shape, rt.Layout(ST.Host, TL.RowMajor, dt))
    pb = rt.ProgramBuilder()
    pb.begin_program("hoisted")
    pb.add_dylib(7, so.read_bytes())
    a = pb.input((6, 5), DT.Float32, TL.RowMajor, ST.Host)
    c = pb.input((6, 5), DT.Float32, TL.RowMajor, ST.Host)
    v = pb.input((9,), DT.Float32, TL.RowMajor, ST.Host)
    s0, s1 = pb.cpu_op(7, "cpu_hoisted_add_rowsum_0a1b2c3d_helper", [a, c], [host((6, 5), DT.Float32), host((6,), DT.Int32)])
    d0, d1 = pb.cpu_op(7, "cpu_hoisted_alias_helper", [v], [host((9,), DT.Float32), host((9,), DT.Float32)])
    (bad,) = pb.cpu_op(7, "no_such_helper", [v], [host((9,), DT.Float32)])
    (bad2,) = pb.cpu_op(8, "cpu_hoisted_alias_helper", [v], [host((9,), DT.Float32)])
    n = pb.unary(0, v)
    for t in (s0, s1, d0, d1, bad, bad2, n):
        pb.output(t)
    pb.end_program()
    binary = rt.Binary.load_from_memory(pb.finish())
    rng = np.random.default_rng(5)
    xa, xc, xv = (rng.standard_normal(s).astype(np.float32) for s in ((6, 5), (6, 5), (9,)))
    f32 = lambda x: rt.create_owned_host_tensor(x, DT.Float32)
    results = {}

    def visit(idx, name, dbg, hook):
        if idx == 0:
            outs = hook.invoke_cpu_op([f32(xa), f32(xc)])
            results[0] = [rt.to_numpy(o) for o in outs]
            assert [o.get_layout() for o in outs] == [rt.Layout(ST.Host, TL.RowMajor, DT.Float32), rt.Layout(ST.Host, TL.RowMajor, DT.Int32)]
            for wrong, msg in (([f32(xa)], "input count mismatch: got 1, expected 2"),
                               ([f32(xa), f32(xc[:5])], "input 1 has the wrong shape"),
                               ([f32(xa), rt.create_owned_host_tensor(xc.astype(np.int32), DT.Int32)], "input 1 has the wrong data type"),
                               ([f32(xa), rt.create_owned_host_tensor(xc.view(np.uint32).astype(np.uint16), DT.BFloat16)], "must have 4-byte elements"),
                               ([f32(xa), rt.create_empty_tensor(None, rt.Layout(ST.Host, TL.Tile, DT.Float32), (6, 5))], "must be a row-major host tensor")):
                with pytest.raises(rt.RuntimeError_, match=msg):
                    hook.invoke_cpu_op(wrong)
        elif idx == 1:
            for _ in range(3):   # two outputs that share one buffer: freed once, every time
                outs = hook.invoke_cpu_op([f32(xv)])
                results[1] = [rt.to_numpy(o) for o in outs]
                del outs
        elif idx == 2:
            with pytest.raises(rt.RuntimeError_, match="could not find requested op"):
                hook.invoke_cpu_op([f32(xv)])
        elif idx == 3:
            with pytest.raises(rt.RuntimeError_, match="could not find dylib corresponding to id: 8"):
                hook.invoke_cpu_op([f32(xv)])
        else:
            with pytest.raises(rt.RuntimeError_, match="opContext must wrap a CpuOp, got EltwiseUnaryOp"):
                hook.invoke_cpu_op([f32(xv)])
    rt.walk_program(binary, 0, visit)
    want = xa + xc
    assert np.array_equal(results[0][0], want)
    rows = np.zeros(6, dtype=np.float32)
    for col in range(5):   # the callee's order of additions
        rows = rows + want[:, col]
    assert np.array_equal(results[0][1], rows.astype(np.int32))
    assert np.array_equal(results[1][0], 2 * xv) and np.array_equal(results[1][1], 2 * xv)


def _damaged_binaries_never_crash_the_reader(seed, cases):
    """Body of the test below, run in a child process: a reader that walks off a damaged buffer would take the
    process down, and that must show as a failed test rather than a dead test run."""
    import random
    rnd = random.Random(seed)
    bases = [programs.c1_matmul(), programs.c4_mlp(tokens=64, hidden=128, ffn=256)]
    loaded = 0
    for _ in range(cases):
        data = bytearray(rnd.choice(bases))
        for _ in range(rnd.choice([1, 1, 2, 4, 8])):
            pos, mode = rnd.randrange(len(data)), rnd.randrange(4)
            data[pos] = (rnd.randrange(256), data[pos] ^ (1 << rnd.randrange(8)), 0xFF, 0)[mode]
        if rnd.random() < 0.1:
            data = data[: rnd.randrange(len(data))]
        try:
            b = rt.Binary.load_from_memory(bytes(data))
            for p in range(min(b.get_num_programs(), 4)):
                b.get_program_name(p), b.get_program_inputs(p), b.get_program_outputs(p)
                b.get_program_ops_as_text(p), b.get_program_ops_as_json(p), b.get_program_inputs_as_json(p)
                rt.walk_program(b, p, lambda i, name, dbg, h: [h.ref_desc(g) for g in h.input_refs() + h.output_refs()] + [h.loc()])
            loaded += 1
        except rt.RuntimeError_:
            pass
    return loaded


def test_damaged_binaries_are_rejected_or_read_but_never_crash():
    # bit flips, byte stamps and truncations of two valid binaries: every access either raises the runtime's error or
    # returns; the offsets a flatbuffer is made of are all checked against the buffer before they are followed
    import subprocess
    import sys
    code = ("import sys; sys.path.insert(0, %r); sys.path.insert(0, %r); import conftest, test_runtime_host as t; "
            "print(sum(t._damaged_binaries_never_crash_the_reader(s, 400) for s in (11, 12, 13)))") % (
        os.path.dirname(os.path.abspath(__file__)), os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, "the reader crashed on a damaged binary (exit %d): %s" % (r.returncode, r.stderr[-400:])
    assert 0 < int(r.stdout.strip().splitlines()[-1]) < 1200   # some damage is harmless, some must be caught


def test_reference_gtest_dump_and_load_float32_tensor(tmp_path):
    # runtime/test/ttnn/gtest/test_tensor_serialization.cpp:40-78 (TestDumpAndLoadFloat32Tensor), its data and its checks
    data = np.array([1.0, 2.5, 3.14159, -1.0, 0.0, 42.0, -3.14159, 1e6, -1e-6], dtype=np.float32).reshape(3, 3)
    original = rt.create_owned_host_tensor(data, DT.Float32)
    path = tmp_path / "test_float32_tensor.bin"
    rt.dump_tensor(original, path)
    loaded = rt.load_tensor(path)
    assert original.get_shape() == loaded.get_shape() == [3, 3]
    assert original.get_dtype() == loaded.get_dtype() == DT.Float32
    a, b = original.get_data_buffer(), loaded.get_data_buffer()
    assert len(a) == len(b) == 36 and a == b


def test_reference_gtest_unsafe_borrowed_host_tensor_aliases_owned_buffer():
    # runtime/test/ttnn/gtest/test_unsafe_borrowed_host_tensor.cpp:26-51 (AliasesOwnedBuffer)
    owned = rt.create_owned_host_tensor(np.array([[1.0, 2.0], [3.0, 4.0]], dtype=np.float32), DT.Float32)
    borrowed = rt.create_unsafe_borrowed_host_tensor(owned)
    assert rt.host_data_ptr(owned) == rt.host_data_ptr(borrowed) != 0
    assert owned.get_shape() == borrowed.get_shape() and owned.get_dtype() == borrowed.get_dtype()
    # one buffer: what is copied into the owner is what the borrower reads
    rt.memcpy_tensor(owned, rt.create_owned_host_tensor(np.full((2, 2), 7.0, dtype=np.float32), DT.Float32))
    assert np.array_equal(rt.to_numpy(borrowed), np.full((2, 2), 7.0, dtype=np.float32))
    # only row-major host tensors have a buffer that can be borrowed this way (runtime/lib/ttnn/runtime.cpp:287-298)
    with pytest.raises(rt.RuntimeError_, match="requires ROW_MAJOR layout"):
        rt.create_unsafe_borrowed_host_tensor(rt.create_empty_tensor(None, rt.Layout(ST.Host, TL.Tile, DT.Float32), (32, 32)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_reference_tensor_buffer_api(dtype):
    # runtime/test/ttnn/python/n150/test_runtime_api.py:22-57 (test_tensor_buffer_api): a borrowed host tensor reports the
    # shape, stride, element size, volume, data type and bytes of the memory it was made from
    import torch
    tdt = getattr(torch, dtype)
    t = torch.randn((64, 128), dtype=tdt)
    rtt = rt.from_torch(t, borrowed=True)
    desc = rtt.get_tensor_desc()
    assert desc.shape == rtt.get_shape() and desc.stride == rtt.get_stride()
    assert desc.dtype == rtt.get_dtype() and desc.item_size == rtt.get_element_size()
    assert rtt.get_shape() == [64, 128] and rtt.get_stride() == list(t.stride())
    assert rtt.get_element_size() == t.element_size() and rtt.get_volume() == t.numel()
    assert rtt.get_dtype() == (DT.Float32 if dtype == "float32" else DT.BFloat16)
    raw = rtt.get_data_buffer()
    assert len(raw) == rtt.get_volume() * rtt.get_element_size()
    assert torch.equal(torch.frombuffer(raw, dtype=tdt).reshape(rtt.get_shape()), t)
