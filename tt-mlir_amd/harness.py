"""execute_fb-style driver: host tensors -> to_layout(get_layout) -> submit -> wait -> to_host(untilize)
(tools/builder/base/builder_runtime.py:529-827).  Golden comparison is left to the caller."""
from . import runtime as rt


def execute(binary, program, torch_inputs, device=None, retain_inputs=False):
    """Run one program on torch CPU inputs; returns the outputs as torch tensors."""
    own = device is None
    dev = device or rt.open_mesh_device()
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
        return res
    finally:
        if own:
            rt.close_mesh_device(dev)
