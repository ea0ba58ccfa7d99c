"""Command-line runner for `.ttnn` binaries in the style of `ttrt` (tools/ttrt/common/{run,read,query}.py).

    python tt-mlir_amd/ttrt.py read  model.ttnn [--section all|version|programs|inputs|outputs|ops|goldens]
    python tt-mlir_amd/ttrt.py run   model.ttnn [--program-index all|N] [--loops N] [--init randn|arange|zeros|ones]
                                     [--seed S] [--enable-golden] [--pcc P] [--atol A] [--rtol R] [--non-zero]
                                     [--save-artifacts] [--artifact-dir DIR] [--result-file FILE] [--benchmark]
    python tt-mlir_amd/ttrt.py query

`run` follows tools/ttrt/common/run.py:534-873: seeded inputs per program (torch.manual_seed, run.py:566), host
tensors -> to_layout(get_layout) -> submit per loop -> wait -> to_host(untilize); with --enable-golden every
operation whose location carries an embedded golden is compared in the post-op hook, and a golden stored for
"output_<i>" is compared with the program's i-th output (run.py:687-731, 799-846).  One record per binary goes to the
result file as {file_path, result: pass|error, exception, program_index, program_results} (run.py:1160-1172); the exit
code is 0 only if every binary passed.  --save-artifacts writes <artifact-dir>/<binary name>/run/program_<i>/
input_<k>.pt and device_output_<k>.pt beside a copy of the binary (tools/ttrt/common/util.py:725-752).
"""
import argparse
import json
import os
import shutil
import sys
import time

import numpy as np

if not __package__:
    # run as a script: the package directory is not a valid module name, so register it as `ttmlir_amd` first
    import importlib.util
    _dir = os.path.dirname(os.path.abspath(__file__))
    if "ttmlir_amd" not in sys.modules:
        _spec = importlib.util.spec_from_file_location("ttmlir_amd", os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir])
        _mod = importlib.util.module_from_spec(_spec)
        sys.modules["ttmlir_amd"] = _mod
        _spec.loader.exec_module(_mod)
    from ttmlir_amd import runtime as rt
    from ttmlir_amd.harness import _pcc
else:
    from . import runtime as rt
    from .harness import _pcc

DT = rt.DataType
_TORCH_OF = None


def _torch_dtype(dt):
    import torch
    global _TORCH_OF
    if _TORCH_OF is None:
        _TORCH_OF = {DT.Float32: torch.float32, DT.Float16: torch.float16, DT.BFloat16: torch.bfloat16, DT.UInt32: torch.int64,
                     DT.UInt16: torch.int32, DT.UInt8: torch.uint8, DT.Int32: torch.int32, DT.Float64: torch.float64,
                     DT.Int64: torch.int64, DT.UInt64: torch.int64, DT.Int16: torch.int16, DT.Int8: torch.int8, DT.Bool: torch.bool}
    # block-float inputs are produced from bf16 values by to_layout
    return _TORCH_OF.get(dt, torch.bfloat16)


def make_input(shape, dtype, init, generator):
    """One host input for `--init`; integer inputs get small non-negative values so that index operands stay in range."""
    import torch
    td = _torch_dtype(dtype)
    n = int(np.prod(shape)) if len(shape) else 1
    if init == "zeros":
        return torch.zeros(shape, dtype=td)
    if init == "ones":
        return torch.ones(shape, dtype=td)
    if init == "arange":
        return torch.arange(n, dtype=torch.float32).reshape(shape).to(td)
    if td.is_floating_point:
        return torch.randn(shape, generator=generator, dtype=torch.float32).to(td)
    if td == torch.bool:
        return torch.randint(0, 2, shape, generator=generator).to(td)
    return torch.randint(0, 8, shape, generator=generator).to(td)


def read_binary(binary, section="all"):
    out = {}
    if section in ("all", "version"):
        ident, version = binary.info()
        out["file_identifier"], out["version"] = ident, version
    n = binary.get_num_programs()
    if section in ("all", "programs"):
        out["programs"] = [{"index": i, "name": binary.get_program_name(i), "private": binary.is_program_private(i)} for i in range(n)]
    if section in ("all", "inputs"):
        out["inputs"] = [binary.get_program_inputs_as_json(i) for i in range(n)]
    if section in ("all", "outputs"):
        out["outputs"] = [binary.get_program_outputs_as_json(i) for i in range(n)]
    if section in ("all", "ops"):
        out["ops"] = [binary.get_program_ops_as_json(i) for i in range(n)]
    if section in ("all", "goldens"):
        gold = []
        for i in range(n):
            locs = [o["loc_info"] for o in binary.get_program_ops_as_json(i)]
            if not binary.is_program_private(i):
                # "input_<k>" / "output_<k>" keys are looked up over the whole binary; list them with the programs a runner runs
                locs += ["input_%d" % k for k in range(len(binary.get_program_inputs(i)))]
                locs += ["output_%d" % k for k in range(len(binary.get_program_outputs(i)))]
            found = []
            for loc in locs:
                g = binary.get_debug_info_golden(loc)
                if g is not None:
                    found.append({"loc": loc, "name": g[0], "shape": list(g[1].shape), "dtype": str(g[1].dtype)})
            gold.append(found)
        out["goldens"] = gold
    return out


def run_program(binary, program, device, args, artifact_dir=None):
    """Runs one program `--loops` times; returns its record for program_results.  Raises on a failed check."""
    import torch
    gen = torch.Generator().manual_seed(args.seed)
    descs = binary.get_program_inputs(program)
    host_inputs = []
    for k, (shape, lay) in enumerate(descs):
        g = binary.get_debug_info_golden("input_%d" % k) if args.enable_golden else None
        if g is not None and tuple(g[1].shape) == tuple(shape):
            host_inputs.append(torch.from_numpy(np.ascontiguousarray(g[1])).to(_torch_dtype(lay.dtype)))
        else:
            host_inputs.append(make_input(shape, lay.dtype, args.init, gen))
    report = {}
    if args.enable_golden:
        def post(idx, name, dbg, hook):
            if hook.program_index() != program:
                return
            loc = hook.loc()
            g = binary.get_debug_info_golden(loc)
            out = hook.output() if g is not None else None
            if out is None:
                return
            got = rt.to_torch(out).float().numpy()
            want = np.asarray(g[1], dtype=np.float32)
            if got.size != want.size:
                report[loc] = {"op": name, "result": "error", "exception": "shape %s vs golden %s" % (got.shape, want.shape)}
                return
            got = got.reshape(want.shape)
            p = _pcc(want, got)
            report[loc] = {"op": name, "golden": g[0], "actual_pcc": p, "expected_pcc": args.pcc,
                           "max_abs": float(np.max(np.abs(got - want))) if want.size else 0.0,
                           "allclose": bool(np.allclose(got, want, rtol=args.rtol, atol=args.atol)),
                           "result": "pass" if p >= args.pcc else "fail"}
        rt.set_post_op_callback(post)
    loops = []
    outs_host = []
    try:
        warm = 1 if args.benchmark else 0
        for it in range(args.loops + warm):
            t0 = time.perf_counter_ns()
            ins = [rt.to_layout(rt.from_torch(t), device, rt.get_layout(binary, program, k)) for k, t in enumerate(host_inputs)]
            t1 = time.perf_counter_ns()
            outs = rt.submit(device, binary, program, ins)
            rt.wait(outs)
            t2 = time.perf_counter_ns()
            outs_host = [rt.to_torch(rt.to_host(o, untilize=True)[0]) for o in outs]
            t3 = time.perf_counter_ns()
            for o in outs:
                rt.deallocate_tensor(o, force=True)
            for t in ins:
                if t.is_allocated():
                    rt.deallocate_tensor(t, force=True)
            if it >= warm:
                loops.append({"loop": it - warm, "inputs_ns": t1 - t0, "submit_ns": t2 - t1, "outputs_ns": t3 - t2,
                              "total_duration_ns": t3 - t0})
    finally:
        if args.enable_golden:
            rt.clear_callbacks()
    rec = {"program_index": program, "name": binary.get_program_name(program), "loops": loops}
    if args.enable_golden:
        for k, y in enumerate(outs_host):
            g = binary.get_debug_info_golden("output_%d" % k)
            if g is None or g[1].size != y.numel():
                continue
            want = np.asarray(g[1], dtype=np.float32)
            got = y.float().numpy().reshape(want.shape)
            p = _pcc(want, got)
            report["output_%d" % k] = {"op": "program output", "golden": g[0], "actual_pcc": p, "expected_pcc": args.pcc,
                                       "max_abs": float(np.max(np.abs(got - want))) if want.size else 0.0,
                                       "allclose": bool(np.allclose(got, want, rtol=args.rtol, atol=args.atol)),
                                       "result": "pass" if p >= args.pcc else "fail"}
        rec["golden_report"] = report
    if artifact_dir:
        folder = os.path.join(artifact_dir, "run", "program_%d" % program)
        os.makedirs(folder, exist_ok=True)
        for k, t in enumerate(host_inputs):
            torch.save(t, os.path.join(folder, "input_%d.pt" % k))
        for k, t in enumerate(outs_host):
            torch.save(t, os.path.join(folder, "device_output_%d.pt" % k))
        if args.enable_golden:
            with open(os.path.join(folder, "golden_results.json"), "w") as f:
                json.dump(report, f, indent=2)
    if args.non_zero:
        for k, y in enumerate(outs_host):
            if not bool(y.float().abs().sum() > 0):
                raise RuntimeError("program %d output %d is all zero" % (program, k))
    bad = [loc for loc, v in report.items() if v["result"] != "pass"]
    if bad:
        raise RuntimeError("golden comparison failed at " + ", ".join(bad))
    return rec


def cmd_run(args):
    results, ok = [], True
    device = None
    try:
        for path in args.binary:
            rec = {"file_path": path, "result": "pass", "exception": "", "program_index": args.program_index,
                   "artifacts": args.artifact_dir if args.save_artifacts else "", "program_results": []}
            try:
                binary = rt.Binary.load_from_path(path)
                if device is None:
                    device = rt.open_mesh_device()
                n = binary.get_num_programs()
                if args.program_index == "all":
                    todo = [i for i in range(n) if not binary.is_program_private(i)]
                else:
                    todo = [int(args.program_index)]
                    if not 0 <= todo[0] < n:
                        raise RuntimeError("program index %d out of range (binary has %d programs)" % (todo[0], n))
                art = None
                if args.save_artifacts:
                    art = os.path.join(args.artifact_dir, os.path.splitext(os.path.basename(path))[0])
                    if args.clean_artifacts and os.path.isdir(art):
                        shutil.rmtree(art)
                    os.makedirs(art, exist_ok=True)
                    shutil.copy(path, art)
                for p in todo:
                    rec["program_results"].append(run_program(binary, p, device, args, art))
                print("PASS: test case=%s" % path)
            except Exception as e:  # every failure becomes a record; the exit code reports it
                rec["result"], rec["exception"], ok = "error", str(e), False
                print("ERROR: test case=%s exception=%s" % (path, e))
            results.append(rec)
    finally:
        if device is not None:
            rt.close_mesh_device(device)
    if args.result_file:
        with open(args.result_file, "w") as f:
            json.dump(results, f, indent=2)
    return 0 if ok else 1


def cmd_read(args):
    for path in args.binary:
        print(json.dumps({"file_path": path, **read_binary(rt.Binary.load_from_path(path), args.section)}, indent=2))
    return 0


def cmd_query(args):
    n = rt.get_num_available_devices()
    info = {"num_devices": n}
    if n:
        dev = rt.open_mesh_device()
        info["device"] = dev.name()
        rt.close_mesh_device(dev)
    print(json.dumps(info, indent=2))
    return 0


def main(argv=None):
    ap = argparse.ArgumentParser(prog="ttrt", description=__doc__.splitlines()[0])
    sub = ap.add_subparsers(dest="cmd", required=True)
    r = sub.add_parser("run")
    r.add_argument("binary", nargs="+")
    r.add_argument("--program-index", default="all")
    r.add_argument("--loops", type=int, default=1)
    r.add_argument("--init", default="randn", choices=["randn", "arange", "zeros", "ones"])
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--enable-golden", action="store_true")
    r.add_argument("--pcc", type=float, default=0.99)
    r.add_argument("--atol", type=float, default=1e-8)
    r.add_argument("--rtol", type=float, default=1e-5)
    r.add_argument("--non-zero", action="store_true")
    r.add_argument("--save-artifacts", action="store_true")
    r.add_argument("--clean-artifacts", action="store_true")
    r.add_argument("--artifact-dir", default=os.path.join(os.getcwd(), "ttrt-artifacts"))
    r.add_argument("--result-file", default="run_results.json")
    r.add_argument("--benchmark", action="store_true", help="one untimed warm-up loop before the timed ones")
    r.set_defaults(fn=cmd_run)
    d = sub.add_parser("read")
    d.add_argument("binary", nargs="+")
    d.add_argument("--section", default="all", choices=["all", "version", "programs", "inputs", "outputs", "ops", "goldens"])
    d.set_defaults(fn=cmd_read)
    q = sub.add_parser("query")
    q.set_defaults(fn=cmd_query)
    args = ap.parse_args(argv)
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
