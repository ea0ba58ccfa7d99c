"""execute_fb-style driver: host tensors -> to_layout(get_layout) -> submit -> wait -> to_host(untilize)
(tools/builder/base/builder_runtime.py:529-827).  With enable_golden the run also checks every operation whose
location has a golden tensor embedded in the binary, through the post-operator hook
(tools/builder/base/builder_runtime.py:353-451; `ttrt run --enable-golden`, tools/ttrt/common/run.py:687-731)."""
import numpy as np

from . import runtime as rt


def _pcc(a, b):
    """Pearson correlation with the special cases of tools/golden/metrics.py:39-115 that matter for a pass / fail
    report: equal tensors -> 1, NaN / Inf masked to 0, constant tensors compared with isclose."""
    a = np.nan_to_num(np.asarray(a, dtype=np.float64).ravel(), nan=0.0, posinf=0.0, neginf=0.0)
    b = np.nan_to_num(np.asarray(b, dtype=np.float64).ravel(), nan=0.0, posinf=0.0, neginf=0.0)
    if a.size == 0 or np.array_equal(a, b):
        return 1.0
    if np.ptp(a) == 0 or np.ptp(b) == 0:
        return 1.0 if np.allclose(a, b, rtol=1e-2, atol=1e-2) else 0.0
    return float(np.corrcoef(a, b)[0, 1])


def execute(binary, program, torch_inputs, device=None, retain_inputs=False, enable_golden=False, pcc=0.99):
    """Run one program on torch CPU inputs; returns the outputs as torch tensors.  With enable_golden returns
    (outputs, report) where report maps op location -> {"name", "pcc", "max_abs", "pass"}."""
    own = device is None
    dev = device or rt.open_mesh_device()
    report = {}
    if enable_golden:
        def post(idx, name, dbg, get_output):
            loc = get_output.loc()
            g = binary.get_debug_info_golden(loc)
            if g is None:
                return
            out = get_output()
            if out is None:
                return
            got = rt.to_torch(out).float().numpy()
            want = np.asarray(g[1], dtype=np.float32)
            if got.size != want.size:
                report[loc] = {"name": g[0], "op": name, "pcc": 0.0, "max_abs": float("inf"), "pass": False,
                               "error": "shape %s vs golden %s" % (got.shape, want.shape)}
                return
            p = _pcc(want, got.reshape(want.shape))
            report[loc] = {"name": g[0], "op": name, "pcc": p, "max_abs": float(np.max(np.abs(got.reshape(want.shape) - want))),
                           "pass": p >= pcc}
        rt.set_post_op_callback(post)
    try:
        ins = []
        for i, t in enumerate(torch_inputs):
            h = rt.from_torch(t)
            ins.append(rt.to_layout(h, dev, rt.get_layout(binary, program, i), retain=retain_inputs))
        outs = rt.submit(dev, binary, program, ins)
        rt.wait(outs)
        res = [rt.to_torch(rt.to_host(o, untilize=True)[0]) for o in outs]
        for o in outs:
            rt.deallocate_tensor(o, force=True)
        return (res, report) if enable_golden else res
    finally:
        if enable_golden:
            rt.clear_callbacks()
        if own:
            rt.close_mesh_device(dev)
