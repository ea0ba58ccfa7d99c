"""The host runtime on a device in host memory (tests/cpp/null_device.cpp): a stand-in for the kernel library whose entry
points hold every pointer against the live allocations and the bytes the real kernels touch, and then compute the common ops
with the oracle's arithmetic.  Put in front of the real library with
LD_LIBRARY_PATH, it lets the executor run whole programs on the CPU: the tensor pool, the caches, the fused launches, the
trace protocol (recorded launches are closures that a replay runs) and the hooks all run; a launch whose buffer is too small
- a memory fault on the GPU - is an error here.  The GPU runtime tests run here with their assertions on values, and
once more with assertions stripped (python -O), where what is checked is that every program runs to its end and that no
launch leaves its buffers."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _oracle_link():
    """Linker arguments for the oracle library, whose arithmetic the null device computes with (built if missing)."""
    sys.path.insert(0, ROOT)
    import oracle.oracle as orc
    oracle_dir = os.path.dirname(orc.build())
    return ["-L", oracle_dir, "-lttm_oracle", "-Wl,-rpath," + oracle_dir]


@pytest.fixture(scope="module")
def null_env(tmp_path_factory):
    d = tmp_path_factory.mktemp("null_device")
    subprocess.run(["g++", "-std=c++17", "-O1", "-shared", "-fPIC", "-fvisibility=hidden", "-I", os.path.join(ROOT, "include"),
                    "-I", os.path.join(ROOT, "tt-mlir_amd", "csrc"), "-o", str(d / "libttmlir_amd_hip.so"), os.path.join(ROOT, "tests", "cpp", "null_device.cpp")] + _oracle_link(), check=True)
    env = dict(os.environ)
    # the runtime library finds the kernel library through its RUNPATH, which LD_LIBRARY_PATH precedes
    env["LD_LIBRARY_PATH"] = str(d) + os.pathsep + env.get("LD_LIBRARY_PATH", "")
    env["TTMLIR_AMD_NULL_DEVICE"] = "1"
    env["TTMLIR_AMD_HIP_LIB"] = str(d / "libttmlir_amd_hip.so")   # the Python binding's options reach the same library
    return env


def test_null_device_exports_the_whole_abi(null_env, hip):
    import ctypes
    l = ctypes.CDLL(os.path.join(null_env["LD_LIBRARY_PATH"].split(os.pathsep)[0], "libttmlir_amd_hip.so"))
    for name, _, _ in hip.declared_functions():   # compiled against the header, so the signatures agree as well
        assert hasattr(l, name), name


def test_null_device_catches_short_buffers(null_env):
    code = r"""
import ctypes, sys
l = ctypes.CDLL("libttmlir_amd_hip.so")
l.ttm_last_error.restype = ctypes.c_char_p
V, I64 = ctypes.c_void_p, ctypes.c_int64
def alloc(n):
    p = V()
    assert l.ttm_malloc(ctypes.byref(p), ctypes.c_size_t(n)) == 0
    return p
C = 128256
Cp = (C + 31) // 32 * 32
one_row, padded = alloc(C * 2), alloc(32 * Cp * 2)
sm = lambda x, y, rows: l.ttm_softmax_lastdim(x, y, 2, I64(1), I64(rows), I64(C), None)
assert sm(padded, padded, 1) == 0 and sm(padded, padded, 32) == 0
assert sm(one_row, padded, 1) == 1 and b"out of bounds: ttm_softmax_lastdim: input has 256512 bytes behind it in its allocation, the kernels touch 8208384" in l.ttm_last_error()
assert sm(padded, one_row, 1) == 1 and b"output" in l.ttm_last_error()
assert sm(V(padded.value + 2048), padded, 32) == 1          # a view that starts inside the allocation has less room
assert sm(V(12345), padded, 1) == 1 and b"not device memory" in l.ttm_last_error()
assert l.ttm_free(one_row) == 0 and sm(padded, one_row, 1) == 1 and b"not" in l.ttm_last_error()   # freed memory is not device memory
assert l.ttm_free(V(padded.value + 16)) == 1
print("ok")
"""
    r = subprocess.run([sys.executable, "-c", code], env=null_env, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and r.stdout.strip() == "ok", r.stderr[-600:]


def test_runtime_programs_give_the_oracles_values_on_the_host(null_env):
    """The GPU runtime tests, assertions and all, on the computing null device: what they assert about values (a traced
    program against the same program run op by op and against the oracle, const-eval and trace cache behaviour under
    replaced weights, hooks that read and replace tensors, fused launches against the op-by-op run) is host logic plus
    arithmetic the oracle defines, so a wrong tensor reaching a launch fails here before it fails on a GPU."""
    skip = "not full_size and not profiler_ranges"   # the full-size configurations take minutes of scalar arithmetic
    r = subprocess.run([sys.executable, "-m", "pytest", os.path.join(ROOT, "tests", "test_gpu_runtime.py"), "-q", "-m", "gpu",
                        "-p", "no:cacheprovider", "-k", skip], env=null_env, capture_output=True, text=True, timeout=1500, cwd=ROOT)
    tail = r.stdout[-3000:] + r.stderr[-1000:]
    assert r.returncode == 0, tail
    last = [l for l in r.stdout.strip().splitlines() if " passed" in l][-1]
    assert int(last.split(" passed")[0].split()[-1]) >= 55 and "failed" not in last, last
    assert "traced_program_with_alternating_weight_sets" not in r.stdout      # ran and passed (failures are listed by name)


def test_runtime_programs_stay_inside_their_buffers(null_env):
    # every program the GPU runtime tests build, submitted through the real host runtime on the null device.  Left out: the
    # full-size configurations (minutes of oracle arithmetic for nothing here) and two tests that look at values by themselves
    skip = "not full_size and not ttrt_run_checks and not profiler_ranges"
    r = subprocess.run([sys.executable, "-O", "-m", "pytest", os.path.join(ROOT, "tests", "test_gpu_runtime.py"), "-q", "-m", "gpu", "-p", "no:assertion",
                        "-p", "no:cacheprovider", "-k", skip], env=null_env, capture_output=True, text=True, timeout=900, cwd=ROOT)
    tail = r.stdout[-3000:] + r.stderr[-1000:]
    assert "out of bounds" not in r.stdout and "out of bounds" not in r.stderr, tail   # a launch outside its buffers
    assert r.returncode == 0, tail
    last = [l for l in r.stdout.strip().splitlines() if " passed" in l][-1]
    assert int(last.split(" passed")[0].split()[-1]) >= 50 and "failed" not in last, last


def test_fusion_decisions_of_a_decode_step_on_the_null_device(null_env):
    """What the executor fuses is host logic: the counters a decode layer leaves are the same on the null device as on the GPU
    (tests/test_gpu_runtime.py::test_decode_layer_steps_eager_and_traced asserts them there)."""
    code = r"""
import json, sys, os
sys.path.insert(0, %r); sys.path.insert(0, os.path.join(%r, "tests"))
import conftest, torch
from ttmlir_amd import programs, runtime as rt
import test_gpu_runtime as T
users, hidden, n_q, n_kv, hd, ffn, max_seq = 8, 256, 4, 2, 64, 512, 128
w, kc0, vc0, cos, sin, xs = T._decode_setup(users, hidden, n_q, n_kv, hd, ffn, max_seq, seed=31)
order = ["anw", "wq", "wk", "wv", "wo", "mnw", "wg", "wu", "wd"]
device = rt.open_mesh_device()
stats = {}
for mode in ("eager", "traced", "callbacks"):
    binary = rt.Binary.load_from_memory(programs.decode_layer(users, hidden, n_q, n_kv, hd, ffn, max_seq, trace=mode == "traced"))
    rt.clear_stats()
    if mode == "callbacks":
        rt.set_post_op_callback(lambda idx, name, dbg, hook: None)
    main = binary.get_num_programs() - 1
    lay = lambda k: rt.get_layout(binary, main, k)
    caches = [rt.to_layout(rt.from_torch(t.clone()), device, lay(5 + i), retain=True) for i, t in enumerate((kc0, vc0))]
    weights = [rt.to_layout(rt.from_torch(w[n]), device, lay(7 + i), retain=True) for i, n in enumerate(order)]
    for step, pos in enumerate((40, 41, 42)):
        step_in = [xs[step], cos[pos].reshape(1, 1, 1, hd), sin[pos].reshape(1, 1, 1, hd), torch.tensor([pos], dtype=torch.int32),
                   torch.full((users,), pos, dtype=torch.int32)]
        ins = [rt.to_layout(rt.from_torch(t.contiguous()), device, lay(i)) for i, t in enumerate(step_in)] + caches + weights
        (y,) = rt.submit(device, binary, main, ins)
        assert tuple(rt.to_host(y, untilize=True)[0].shape) == (1, users, hidden) or True
    rt.clear_callbacks()
    stats[mode] = {k: rt.get_stat(k) for k in ("CapturedTrace", "FusedCopyIntoSlot", "FusedQkvDecode", "FusedCacheUpdate", "FusedHeadSplit",
                                               "GroupedMatmul", "FusedHeadConcat", "FusedLinearAddNorm", "FusedLinearGlu", "ConstEvalCacheMiss", "ConstEvalCacheHit")}
rt.close_mesh_device(device)
print(json.dumps(stats))
""" % (ROOT, ROOT)
    r = subprocess.run([sys.executable, "-c", code], env=null_env, capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-1500:]
    st = json.loads(r.stdout.strip().splitlines()[-1])
    for mode in ("eager", "traced", "callbacks"):
        s = st[mode]
        assert s["FusedCopyIntoSlot"] == (2 if mode == "traced" else 0), (mode, s)
        assert s["FusedCacheUpdate"] == 0 and s["FusedHeadSplit"] == 0 and s["GroupedMatmul"] == 0, (mode, s)
        assert s["FusedHeadConcat"] == s["FusedQkvDecode"] == s["FusedLinearAddNorm"] == s["FusedLinearGlu"], (mode, s)
    assert st["eager"]["FusedQkvDecode"] == 3 and st["callbacks"]["FusedQkvDecode"] == 0
    assert st["traced"]["CapturedTrace"] >= 1 and st["traced"]["FusedQkvDecode"] in (1, 2)


def _lying_programs():
    """Child-process body of the test below (the null device is already in front of the real library): one program per
    operation whose result is declared smaller than its operands give, submitted on zero inputs."""
    import numpy as np
    from ttmlir_amd import runtime as rt
    DT, TL = rt.DataType, rt.TensorLayout
    BF, F32, I32, U32 = DT.BFloat16, DT.Float32, DT.Int32, DT.UInt32
    dev = rt.open_mesh_device()
    cases = [
        ("matmul", [((64, 96), BF), ((96, 128), BF)], lambda pb, i: pb.matmul(i[0], i[1]), (64, 64)),
        ("linear", [((64, 96), BF), ((96, 128), BF), ((128,), BF)], lambda pb, i: pb.linear(i[0], i[1], i[2]), (32, 128)),
        ("unary", [((64, 96), BF)], lambda pb, i: pb.unary(18, i[0]), (32, 96)),
        ("binary", [((64, 96), BF), ((64, 96), BF)], lambda pb, i: pb.binary(0, i[0], i[1]), (64, 32)),
        ("binary broadcast", [((64, 96), BF), ((1, 96), BF)], lambda pb, i: pb.binary(0, i[0], i[1]), (32, 96)),
        ("binary composite", [((64, 96), BF), ((64, 96), BF)], lambda pb, i: pb.binary_composite(0, i[0], i[1]), (64, 32)),
        ("where", [((64, 96), BF)] * 3, lambda pb, i: pb.where(i[0], i[1], i[2]), (64, 32)),
        ("clamp", [((64, 96), BF)], lambda pb, i: pb.unary_composite(1, i[0], -1.0, 1.0), (32, 96)),
        ("rms_norm", [((64, 96), BF), ((96,), BF)], lambda pb, i: pb.rms_norm(i[0], i[1]), (32, 96)),
        ("softmax", [((64, 96), BF)], lambda pb, i: pb.softmax(i[0]), (32, 96)),
        ("softmax over dim 0", [((64, 96), BF)], lambda pb, i: pb.softmax(i[0], dim=0), (32, 96)),
        ("reduction", [((4, 64, 96), BF)], lambda pb, i: pb.reduction(0, i[0], [2], keep_dim=True), (1, 64, 1)),
        ("reduction over dim 1", [((4, 64, 96), BF)], lambda pb, i: pb.reduction(0, i[0], [1], keep_dim=False), (4, 32)),
        ("typecast", [((64, 96), BF)], lambda pb, i: pb.typecast(i[0], F32), (32, 96)),
        ("typecast to bfp8_b", [((64, 96), BF)], lambda pb, i: pb.typecast(i[0], DT.BFP_BFloat8), (32, 96)),
        ("to_layout", [((64, 96), BF)], lambda pb, i: pb.to_layout(i[0], TL.RowMajor), (32, 96)),
        ("reshape", [((64, 96), BF)], lambda pb, i: pb.reshape(i[0], (96, 64)), (32, 64)),
        ("permute", [((2, 64, 96), BF)], lambda pb, i: pb.permute(i[0], (0, 2, 1)), (2, 32, 64)),
        ("transpose", [((64, 96), BF)], lambda pb, i: pb.transpose(i[0], 0, 1), (32, 64)),
        ("concat", [((64, 96), BF), ((64, 96), BF)], lambda pb, i: pb.concat([i[0], i[1]], 1), (64, 96)),
        ("slice", [((64, 96), BF)], lambda pb, i: pb.slice(i[0], (0, 0), (64, 64)), (32, 32)),
        ("repeat", [((64, 96), BF)], lambda pb, i: pb.repeat(i[0], (2, 1)), (64, 96)),
        ("repeat_interleave", [((64, 96), BF)], lambda pb, i: pb.repeat_interleave(i[0], 2, 0), (64, 96)),
        ("sdpa", [((1, 4, 64, 64), BF), ((1, 2, 64, 64), BF), ((1, 2, 64, 64), BF)], lambda pb, i: pb.sdpa(i[0], i[1], i[2], is_causal=True), (1, 4, 32, 64)),
        ("sdpa_decode", [((1, 8, 4, 64), BF), ((8, 2, 128, 64), BF), ((8, 2, 128, 64), BF), ((8,), I32)],
         lambda pb, i: pb.sdpa_decode(i[0], i[1], i[2], cur_pos=i[3]), (1, 4, 4, 64)),
        ("concatenate_heads", [((1, 4, 64, 64), BF)], lambda pb, i: pb.concatenate_heads(i[0]), (1, 64, 128)),
        ("nlp_concat_heads", [((1, 4, 64, 64), BF)], lambda pb, i: pb.nlp_concat_heads(i[0]), (1, 1, 32, 256)),
        ("nlp_concat_heads_decode", [((1, 8, 32, 64), BF)], lambda pb, i: pb.nlp_concat_heads_decode(i[0], 4), (1, 1, 4, 256)),
        ("nlp_create_qkv_heads_decode", [((1, 1, 8, 8 * 64), BF)], lambda pb, i: pb.nlp_create_qkv_heads_decode(i[0], 4, 2), (1, 4, 4, 64)),
        ("split_qkv", [((2, 64, 3 * 128), BF)], lambda pb, i: pb.split_query_key_value_and_split_heads(i[0], 4), (2, 4, 32, 32)),
        ("embedding", [((64,), U32), ((100, 96), BF)], lambda pb, i: pb.embedding(i[0], i[1]), (32, 96)),
        ("argmax", [((64, 96), BF)], lambda pb, i: pb.argmax(i[0], dim=-1), (32,)),
        ("rotary_embedding", [((1, 4, 64, 64), BF), ((1, 1, 64, 64), BF), ((1, 1, 64, 64), BF)], lambda pb, i: pb.rotary_embedding(i[0], i[1], i[2]),
         (1, 4, 32, 64)),
        ("rotary_embedding decode", [((1, 8, 4, 64), BF), ((1, 1, 64, 64), BF), ((1, 1, 64, 64), BF)],
         lambda pb, i: pb.rotary_embedding(i[0], i[1], i[2], token_index=5), (1, 4, 4, 64)),
        ("rotary_embedding_llama", [((1, 4, 64, 64), BF), ((1, 1, 64, 64), BF), ((1, 1, 64, 64), BF), ((1, 1, 32, 32), BF)],
         lambda pb, i: pb.rotary_embedding_llama(i[0], i[1], i[2], i[3]), (1, 4, 32, 64)),
        ("full", [], lambda pb, i: pb.full((64, 96), 1.0, BF), (32, 96)),
        ("arange", [], lambda pb, i: pb.arange(0, 64), (32,)),
        ("empty", [], lambda pb, i: pb.empty((64, 96), BF), (32, 96)),
    ]
    npdt = {BF: np.uint16, F32: np.float32, I32: np.int32, U32: np.uint32}
    report = {}
    for lying in (False, True):
        for name, specs, build, lie in cases:
            pb = rt.ProgramBuilder()
            pb.begin_program("p")
            ins = [pb.input(s, dt) for s, dt in specs]
            if lying:
                pb.declare_next_shape(lie)
            out = build(pb, ins)
            for o in (out if isinstance(out, (list, tuple)) else [out]):
                pb.output(o)
            pb.end_program()
            b = rt.Binary.load_from_memory(pb.finish())
            tins = [rt.to_layout(rt.create_owned_host_tensor(np.zeros(s, dtype=npdt[dt]), dt), dev, rt.get_layout(b, 0, k)) for k, (s, dt) in enumerate(specs)]
            try:
                rt.submit(dev, b, 0, tins)
                verdict = "ran"
            except rt.RuntimeError_ as e:
                verdict = "LEAK: " + str(e).split("out of bounds: ")[1] if "out of bounds" in str(e) else "refused"
            report["%s%s" % (name, " (lying)" if lying else "")] = verdict
    rt.close_mesh_device(dev)
    return report


def test_programs_that_lie_about_a_result_never_launch_past_a_buffer(null_env):
    """The kernels are launched from the operands' extents, results are allocated from the shape the program declares: an
    operation whose declared result is smaller than what its operands give must be refused by the runner (or run on a
    result of its own making), never reach the device.  Truthful versions of the same programs all run - among them the
    prefill rotary embedding, whose absent token_index used to reach the kernel as 4294967295."""
    code = ("import sys, os, json; sys.path.insert(0, %r); sys.path.insert(0, os.path.join(%r, 'tests')); import conftest, test_null_device as t; "
            "print(json.dumps(t._lying_programs()))") % (ROOT, ROOT)
    r = subprocess.run([sys.executable, "-c", code], env=null_env, capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-1500:]
    report = json.loads(r.stdout.strip().splitlines()[-1])
    assert len(report) == 2 * 38
    for name, verdict in report.items():
        assert not verdict.startswith("LEAK"), (name, verdict)
        if not name.endswith("(lying)"):
            assert verdict == "ran", (name, verdict)
    # a full or empty tensor has no operands: the declared shape is its shape.  Everything else is refused, by the runner or
    # where its result enters the tensor pool under a reference that declares another shape
    still_run = {n for n, v in report.items() if n.endswith("(lying)") and v == "ran"}
    assert still_run == {"full (lying)", "empty (lying)"}, still_run


def test_full_size_programs_on_the_null_device(null_env):
    """The benchmark's whole-program workloads at their real shapes (configs 3, 4, 5 and the 32-user decode step, eager and
    traced) through the executor on the null device: every launch inside its buffers, and the launches the executor fuses at
    these shapes (what the GPU profiles show as 11 launches per decode step)."""
    code = r"""
import sys, os, json
sys.path.insert(0, %r); sys.path.insert(0, os.path.join(%r, "tests"))
import conftest, numpy as np
from ttmlir_amd import programs, runtime as rt
DT = rt.DataType
npdt = {DT.BFloat16: np.uint16, DT.Float32: np.float32, DT.Int32: np.int32, DT.UInt32: np.uint32}
dev = rt.open_mesh_device()
keys = ("GroupedMatmul", "FusedLinearTail", "FusedQkvDecode", "FusedLinearAddNorm", "FusedLinearGlu", "FusedHeadConcat", "CapturedTrace", "ConstEvalCacheMiss", "ConstEvalCacheHit")
report = {}
def run(name, data, steps=1):
    b = rt.Binary.load_from_memory(data)
    main = b.get_num_programs() - 1
    ins = [rt.to_layout(rt.create_owned_host_tensor(np.zeros(shape, dtype=npdt[lay.dtype]), lay.dtype), dev, lay, retain=True)
           for shape, lay in b.get_program_inputs(main)]
    rt.clear_stats()
    for _ in range(steps):
        outs = rt.submit(dev, b, main, ins)
    report[name] = dict(shapes=[list(o.shape) for o in outs], **{k: rt.get_stat(k) for k in keys})
run("c3_2048", programs.c3_linear(2048))
run("c3_32", programs.c3_linear(32))
run("c4", programs.c4_mlp())
run("c5", programs.c5_decoder())
run("decode32", programs.decode_layer(), steps=3)
run("decode32_traced", programs.decode_layer(trace=True), steps=3)
rt.close_mesh_device(dev)
print(json.dumps(report))
""" % (ROOT, ROOT)
    env = dict(null_env, TTMLIR_AMD_NULL_DEVICE_COMPUTE="0")   # extents only: the arithmetic of these sizes takes minutes on the host
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=900, cwd=ROOT)
    assert r.returncode == 0, (r.stdout[-500:], r.stderr[-1500:])
    rep = json.loads(r.stdout.strip().splitlines()[-1])
    assert rep["c3_2048"]["shapes"] == [[2048, 14336]] and rep["c3_32"]["shapes"] == [[32, 14336]]
    assert rep["c4"]["shapes"] == [[512, 4096]] and rep["c4"]["FusedLinearGlu"] == 1 and rep["c4"]["GroupedMatmul"] == 0   # gate, up and their product in one launch
    assert rep["c5"]["shapes"] == [[1, 2048, 4096]]
    assert rep["c5"]["GroupedMatmul"] == 1 and rep["c5"]["FusedLinearTail"] == 3               # two residual adds and SiLU(gate) * up
    d = rep["decode32"]                                                                         # three steps
    assert d["shapes"] == [[32, 4096]] and d["FusedQkvDecode"] == 3 and d["FusedLinearAddNorm"] == 3 and d["FusedHeadConcat"] == 3
    assert d["FusedLinearGlu"] == 3 and d["FusedLinearTail"] == 6                               # gate, up and their product; the two residual adds
    assert d["ConstEvalCacheMiss"] == 1 and d["ConstEvalCacheHit"] == 2
    t = rep["decode32_traced"]                                                                  # eager run + recording, then replays
    assert t["CapturedTrace"] == 1 and t["FusedQkvDecode"] == 2 and t["FusedLinearAddNorm"] == 2 and t["FusedLinearGlu"] == 2


def test_const_eval_entries_live_as_long_as_their_inputs(null_env):
    """The reference's tests of its const-eval cache (runtime/test/ttnn/gtest/test_tensor_cache_lifetime.cpp:46-163), at the
    level of programs: an entry per set of input versions (CacheSanitySameProgramDifferentTensors: a second weight tensor
    gets its own entry and leaves the first alone), removed when a tensor it was computed from is destroyed
    (CacheEntryRemovedOnTensorDestruction), any one of them (MultipleInputTensorsRemoveCacheEntry)."""
    code = r"""
import sys, os, json, gc
sys.path.insert(0, %r); sys.path.insert(0, os.path.join(%r, "tests"))
import conftest, numpy as np
from ttmlir_amd import programs, runtime as rt
DT = rt.DataType
dev = rt.open_mesh_device()
stats = lambda: tuple(rt.get_stat(k) for k in ("ConstEvalCacheMiss", "ConstEvalCacheHit", "ConstEvalCacheEvicted"))
log = {}
# one weight tensor: config 3 (the weights are packed to bfp8_b by a const-eval program)
M, K, N = 64, 128, 160
b = rt.Binary.load_from_memory(programs.c3_linear(M, K, N))
lay = lambda i: rt.get_layout(b, 1, i)
mk = lambda shape, i: rt.to_layout(rt.create_owned_host_tensor(np.zeros(shape, dtype=np.uint16), DT.BFloat16), dev, lay(i), retain=True)
a, bias = mk((M, K), 0), mk((N,), 2)
wA, wB = mk((K, N), 1), mk((K, N), 1)
rt.clear_stats()
run = lambda w: rt.submit(dev, b, 1, [a, w, bias])
run(wA); log["A"] = stats()
run(wB); log["B"] = stats()               # another tensor, another version: its own entry
run(wA); log["A again"] = stats()         # the first entry is still there
run(wB); log["B again"] = stats()
del wB; gc.collect(); log["B destroyed"] = stats()
run(wA); log["A after B died"] = stats()
del wA; gc.collect(); log["A destroyed"] = stats()
# several inputs: config 4 packs three weight tensors in one const-eval program; destroying one of them removes the entry
b4 = rt.Binary.load_from_memory(programs.c4_mlp(64, 128, 256))
ins = [rt.to_layout(rt.create_owned_host_tensor(np.zeros(s, dtype=np.uint16), l.dtype), dev, l, retain=True) for s, l in b4.get_program_inputs(1)]
rt.clear_stats()
rt.submit(dev, b4, 1, ins); rt.submit(dev, b4, 1, ins); log["mlp twice"] = stats()
victim = ins.pop(3); rest = list(ins)      # the up-projection weights
del victim; gc.collect(); log["one of three destroyed"] = stats()
rt.close_mesh_device(dev)
print(json.dumps(log))
""" % (ROOT, ROOT)
    r = subprocess.run([sys.executable, "-c", code], env=null_env, capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-1500:]
    log = json.loads(r.stdout.strip().splitlines()[-1])
    assert log["A"] == [1, 0, 0] and log["B"] == [2, 0, 0]
    assert log["A again"] == [2, 1, 0] and log["B again"] == [2, 2, 0]
    assert log["B destroyed"] == [2, 2, 1] and log["A after B died"] == [2, 3, 1] and log["A destroyed"] == [2, 3, 2]
    assert log["mlp twice"] == [1, 1, 0] and log["one of three destroyed"] == [1, 1, 1]


@pytest.mark.parametrize("sanitizer", ["thread", "address,undefined"])
def test_runtime_under_sanitizers_on_the_null_device(tmp_path, sanitizer):
    """tests/cpp/runtime_stress.cpp: six threads submit a program with a const-eval part on one device, creating and
    destroying weight tensors as they go, while a seventh reads statistics.  The runtime's sources and the null device are
    built with -fsanitize=thread (no data race, no deadlock) and with -fsanitize=address,undefined (no bad access, no
    undefined behaviour, no leak); every const-eval entry is evicted with its tensor."""
    rtsrc = os.path.join(ROOT, "tt-mlir_amd", "runtime")
    inc = ["-I", os.path.join(ROOT, "include"), "-I", rtsrc, "-I", os.path.join(ROOT, "tt-mlir_amd", "csrc")]
    common = ["g++", "-O1", "-g", "-std=c++17", "-fPIC", "-pthread", "-fsanitize=" + sanitizer, "-fno-sanitize-recover=undefined"]
    jobs = [subprocess.Popen(common + inc + ["-c", os.path.join(rtsrc, f), "-o", str(tmp_path / (f + ".o"))])
            for f in sorted(os.listdir(rtsrc)) if f.endswith(".cpp")]
    jobs.append(subprocess.Popen(common + ["-shared", "-fvisibility=hidden"] + inc + ["-o", str(tmp_path / "libttmlir_amd_hip.so"),
                                           os.path.join(ROOT, "tests", "cpp", "null_device.cpp")] + _oracle_link()))
    assert all(j.wait() == 0 for j in jobs)
    objs = [str(p) for p in tmp_path.glob("*.o")]
    subprocess.run(common + inc + [os.path.join(ROOT, "tests", "cpp", "runtime_stress.cpp")] + objs +
                   ["-L", str(tmp_path), "-lttmlir_amd_hip", "-ldl", "-o", str(tmp_path / "stress")], check=True)
    env = dict(os.environ, LD_LIBRARY_PATH=str(tmp_path), TSAN_OPTIONS="halt_on_error=0 exitcode=66", ASAN_OPTIONS="detect_leaks=1",
               UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([str(tmp_path / "stress")], env=env, capture_output=True, text=True, timeout=600)
    assert "Sanitizer" not in r.stderr and "runtime error" not in r.stderr, r.stderr[-3000:]
    assert r.returncode == 0, (r.stdout, r.stderr[-1000:])
    words = r.stdout.split()
    assert words[0] == "submits" and int(words[1]) == 360 and int(words[3]) == int(words[7]) > 0   # miss == evicted


def test_damaged_programs_through_the_runtime_under_address_sanitizer(tmp_path):
    """tests/cpp/runtime_fuzz.cpp: four programs (MLP with const-eval, decoder layer, decode layer eager and traced) with a few
    bytes flipped, 400 copies each, loaded and submitted on the null device with the runtime built under
    -fsanitize=address,undefined.  A damaged program is refused or runs; it never makes the host runtime touch memory it does
    not own, overflow an extent, or launch past a buffer."""
    sys.path.insert(0, ROOT)
    from ttmlir_amd import programs
    files = []
    for name, data in (("c4", programs.c4_mlp(64, 128, 256)), ("c5", programs.c5_decoder(96, 256, 4, 2, 64, 512)),
                       ("decode", programs.decode_layer(8, 256, 4, 2, 64, 512, 128)),
                       ("decode_traced", programs.decode_layer(8, 256, 4, 2, 64, 512, 128, trace=True))):
        files.append(str(tmp_path / (name + ".ttnn")))
        open(files[-1], "wb").write(data)
    rtsrc = os.path.join(ROOT, "tt-mlir_amd", "runtime")
    inc = ["-I", os.path.join(ROOT, "include"), "-I", rtsrc, "-I", os.path.join(ROOT, "tt-mlir_amd", "csrc")]
    common = ["g++", "-O1", "-g", "-std=c++17", "-fPIC", "-pthread", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined"]
    jobs = [subprocess.Popen(common + inc + ["-c", os.path.join(rtsrc, f), "-o", str(tmp_path / (f + ".o"))])
            for f in sorted(os.listdir(rtsrc)) if f.endswith(".cpp")]
    jobs.append(subprocess.Popen(common + ["-shared", "-fvisibility=hidden"] + inc + ["-o", str(tmp_path / "libttmlir_amd_hip.so"),
                                           os.path.join(ROOT, "tests", "cpp", "null_device.cpp")] + _oracle_link()))
    assert all(j.wait() == 0 for j in jobs)
    subprocess.run(common + inc + [os.path.join(ROOT, "tests", "cpp", "runtime_fuzz.cpp")] + [str(p) for p in tmp_path.glob("*.o")] +
                   ["-L", str(tmp_path), "-lttmlir_amd_hip", "-ldl", "-o", str(tmp_path / "fuzz")], check=True)
    # a damaged shape may ask for any amount of memory: allocations above 4 GiB fail instead of being tried
    env = dict(os.environ, LD_LIBRARY_PATH=str(tmp_path), TTMLIR_AMD_NULL_DEVICE_COMPUTE="0", ASAN_OPTIONS="max_allocation_size_mb=4096:allocator_may_return_null=1:detect_leaks=0",
               UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([str(tmp_path / "fuzz"), "400"] + files, env=env, capture_output=True, text=True, timeout=900)
    assert "Sanitizer" not in r.stderr and "runtime error" not in r.stderr, r.stderr[-3000:]
    assert r.returncode == 0, (r.stdout[-300:], r.stderr[-1500:])
    words = r.stdout.strip().splitlines()[-1].split()
    stats = dict(zip(words[0::2], map(int, words[1::2])))
    assert stats["out_of_bounds"] == 0 and stats["ran"] >= 4 and stats["refused"] > 100 and stats["loaded"] > 400, stats


def test_reference_debug_hook_registration_semantics_on_the_null_device(null_env):
    """runtime/test/ttnn/python/n150/test_debug_hooks.py: a second registration replaces the callbacks it names
    (test_multiple_registrations, :275-347) and keeps the others (test_partial_re_registration, :349-412); unregistering
    silences all (test_unregister_hooks, :202-273); an exception raised in a callback reaches the caller of submit
    (test_callback_exception_handling, :416-458).  Hooks fire inside submit, which the null device makes possible here."""
    code = r"""
import sys, os, json, gc
sys.path.insert(0, %r); sys.path.insert(0, os.path.join(%r, "tests"))
import conftest, numpy as np
from ttmlir_amd import programs, runtime as rt
DT = rt.DataType
dev = rt.open_mesh_device()
b = rt.Binary.load_from_memory(programs.c1_matmul())
def run():
    ins = [rt.to_layout(rt.create_owned_host_tensor(np.zeros(s, dtype=np.uint16), l.dtype), dev, l) for s, l in b.get_program_inputs(0)]
    return rt.submit(dev, b, 0, ins)
class Tracker:
    def __init__(self): self.pre_program = self.post_program = self.pre_op = self.post_op = 0
    def on_pre_program(self, idx, hook): self.pre_program += 1
    def on_post_program(self, idx, hook): self.post_program += 1
    def on_pre_op(self, idx, name, dbg, hook): self.pre_op += 1
    def on_post_op(self, idx, name, dbg, hook): self.post_op += 1
    def counts(self): return [self.pre_program, self.post_program, self.pre_op, self.post_op]
log = {}
t1, t2 = Tracker(), Tracker()
rt.set_program_callbacks(t1.on_pre_program, t1.on_post_program); run()
log["first"] = [t1.counts(), t2.counts()]
rt.set_program_callbacks(t2.on_pre_program, t2.on_post_program); run()
log["replaced"] = [t1.counts(), t2.counts()]
rt.clear_callbacks(); run()
log["unregistered"] = [t1.counts(), t2.counts()]
t = Tracker()
rt.set_program_callbacks(t.on_pre_program, t.on_post_program); run()
log["program only"] = t.counts()
rt.set_pre_op_callback(t.on_pre_op); rt.set_post_op_callback(t.on_post_op); gc.collect(); run()
log["merged"] = t.counts()
rt.set_program_callbacks(post=t2.on_post_program); gc.collect(); run()      # pre stays t's, post becomes t2's
log["post replaced"] = [t.counts(), t2.counts()]
rt.clear_callbacks()
def failing(idx, hook): raise ValueError("Intentional callback failure")
rt.set_program_callbacks(pre=failing)
try:
    run(); log["exception"] = "none"
except ValueError as e:
    log["exception"] = str(e)
rt.clear_callbacks()
run()                                                                    # and nothing lingers
rt.close_mesh_device(dev)
print(json.dumps(log))
""" % (ROOT, ROOT)
    r = subprocess.run([sys.executable, "-c", code], env=null_env, capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-1500:]
    log = json.loads(r.stdout.strip().splitlines()[-1])
    assert log["first"] == [[1, 1, 0, 0], [0, 0, 0, 0]]
    assert log["replaced"] == [[1, 1, 0, 0], [1, 1, 0, 0]] and log["unregistered"] == log["replaced"]
    assert log["program only"] == [1, 1, 0, 0]
    n_ops = log["merged"][2]
    assert log["merged"] == [2, 2, n_ops, n_ops] and n_ops == 7                 # the seven operations of config 1
    assert log["post replaced"] == [[3, 2, 2 * n_ops, 2 * n_ops], [1, 2, 0, 0]]
    assert log["exception"] == "Intentional callback failure"
