"""`.ttnn` programs of the benchmark configurations, written with the ProgramBuilder.

The reference produces these binaries with its compiler (ttmlir-opt + ttmlir-translate); none is
checked in, so each configuration is rebuilt here op by op in the form the compiler emits:
weights enter as bf16 device tensors and are converted to block-float by a private const-eval
program reached through ttcore.load_cached (TTNNWeightDtypeConversion.cpp:102-131,
test/ttmlir/Silicon/TTNN/n150/mixed_precision/linear.mlir:9); inputs are expected in
Device / Tile / bf16 layout, which callers obtain with to_layout(get_layout(...)).
"""
import numpy as np

from . import runtime as rt

DT, TL, ST = rt.DataType, rt.TensorLayout, rt.StorageType
# EltwiseUnaryOpType / EltwiseBinaryOpType / ReductionOpType values
UNARY = dict(abs=0, ceil=1, cos=2, floor=3, gelu=4, isfinite=5, logical_not=6, neg=7, relu=8, sqrt=9, rsqrt=10,
             sigmoid=11, sin=12, reciprocal=13, sign=14, tan=15, tanh=16, atan=17, exp=18, erf=19, erfc=20, log=21,
             expm1=22, leaky_relu=23, relu6=25, silu=26, hardsigmoid=27, mish=28, acos=29, asin=30, asinh=31)
UNARY_COMPOSITE = dict(cbrt=0, clamp_scalar=1, log1p=3)
BINARY = dict(add=0, multiply=1, subtract=3, eq=4, ne=5, ge=6, gt=7, le=8, lt=9, divide=10)
REDUCE = dict(sum=0, mean=1, max=2, min=3)
BINARY_COMPOSITE = dict(maximum=0, minimum=1, remainder=2, pow=3, atan2=4)


def _consteval_pack(pb, name, shapes_dtypes):
    """Private program: typecast each bf16 weight to its block-float dtype.  Returns (index, out descs)."""
    pb.begin_program(name, private=True)
    outs = []
    for shape, dtype in shapes_dtypes:
        w = pb.input(shape, DT.BFloat16)
        o = pb.typecast(w, dtype)
        pb.output(o)
        outs.append((tuple(shape), rt.Layout(ST.Device, TL.Tile, dtype)))
    return pb.end_program(), outs


def c1_matmul():
    """Config 1: to_layout(TILE) -> matmul [256,512] x [512,256] -> to_layout(ROW_MAJOR); inputs on the host."""
    pb = rt.ProgramBuilder()
    pb.begin_program("c1_matmul")
    a = pb.input((256, 512), DT.BFloat16, TL.RowMajor, ST.Host)
    b = pb.input((512, 256), DT.BFloat16, TL.RowMajor, ST.Host)
    at = pb.to_layout(pb.to_device(a), TL.Tile)
    bt = pb.to_layout(pb.to_device(b), TL.Tile)
    c = pb.matmul(at, bt)
    out = pb.from_device(pb.to_layout(c, TL.RowMajor))
    pb.output(out)
    pb.output(at)      # the tilized operand, so the layout can be checked bit-exactly
    pb.end_program()
    return pb.finish()


def c3_linear(M, K=4096, N=14336, weight_dtype=DT.BFP_BFloat8, activation="gelu", program_config=None):
    """Config 3: linear with block-float weights (packed once by a const-eval program), bias + GELU.
    program_config: optional (kind, fused UnaryOpType or -1) written as the op's matmul_program_config."""
    pb = rt.ProgramBuilder()
    ce, ce_outs = _consteval_pack(pb, "c3_linear_const_eval_0", [((K, N), weight_dtype)])
    pb.begin_program("c3_linear")
    a = pb.input((M, K), DT.BFloat16)
    w = pb.input((K, N), DT.BFloat16)
    bias = pb.input((N,), DT.BFloat16)
    (wq,) = pb.load_cached(ce, "c3_linear_const_eval_0", [w], ce_outs)
    if program_config is not None:
        pb.set_matmul_program_config(*program_config)
    y = pb.linear(a, wq, bias, activation=activation)
    pb.output(y)
    pb.end_program()
    return pb.finish()


def _bf16_bits(a):
    """float32 array -> bf16 bit patterns, round to nearest even."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def _mlp(pb, x, norm_w, wg, wu, wd, eps, goldens=None):
    """goldens: optional {"norm" | "gate" | "up" | "product" | "down": float32 array}; each is embedded as the
    expected bf16 output of the operation that computes it (DebugInfo.golden_info, keyed by the op's location)."""
    def mark(key):
        if goldens and key in goldens:
            pb.golden(pb.last_op_loc(), _bf16_bits(goldens[key]), DT.BFloat16, key)
    h = pb.rms_norm(x, norm_w, 0, eps)
    mark("norm")
    g = pb.linear(h, wg, 0, activation="silu")
    mark("gate")
    u = pb.matmul(h, wu)
    mark("up")
    m = pb.binary(BINARY["multiply"], g, u)
    mark("product")
    pb.deallocate(g)
    pb.deallocate(u)
    d = pb.matmul(m, wd)
    mark("down")
    pb.deallocate(m)
    return d


def c4_mlp(tokens=512, hidden=4096, ffn=14336, eps=1e-5, goldens=None):
    """Config 4: RMSNorm -> gate/up (bfp8_b) -> SiLU(gate)*up -> down (bfp4_b).  goldens: see _mlp."""
    pb = rt.ProgramBuilder()
    ce, ce_outs = _consteval_pack(pb, "c4_mlp_const_eval_0", [((hidden, ffn), DT.BFP_BFloat8), ((hidden, ffn), DT.BFP_BFloat8),
                                                             ((ffn, hidden), DT.BFP_BFloat4)])
    pb.begin_program("c4_mlp")
    x = pb.input((tokens, hidden), DT.BFloat16)
    nw = pb.input((hidden,), DT.BFloat16)
    wg, wu, wd = pb.input((hidden, ffn), DT.BFloat16), pb.input((hidden, ffn), DT.BFloat16), pb.input((ffn, hidden), DT.BFloat16)
    qg, qu, qd = pb.load_cached(ce, "c4_mlp_const_eval_0", [wg, wu, wd], ce_outs)
    pb.output(_mlp(pb, x, nw, qg, qu, qd, eps, goldens))
    # goldens named "input_<k>" / "output_<k>" travel under that name: a runner feeds the former and checks the latter
    for key, value in (goldens or {}).items():
        if key.startswith(("input_", "output_")):
            pb.golden(key, _bf16_bits(value), DT.BFloat16, key)
    pb.end_program()
    return pb.finish()


def c5_decoder(seq=2048, hidden=4096, n_q=32, n_kv=8, head_dim=128, ffn=14336, eps=1e-5):
    """Config 5: Llama-3-8B-shaped decoder layer, batch 1 prefill (op mix of
    test/ttmlir/models/single_blocks_and_layers/llama_3_8b_prefill_layer.mlir:54-304 without rotary embedding)."""
    pb = rt.ProgramBuilder()
    dq, dkv = n_q * head_dim, n_kv * head_dim
    ce, ce_outs = _consteval_pack(pb, "c5_decoder_const_eval_0", [
        ((hidden, dq), DT.BFP_BFloat8), ((hidden, dkv), DT.BFP_BFloat8), ((hidden, dkv), DT.BFP_BFloat8),
        ((dq, hidden), DT.BFP_BFloat8), ((hidden, ffn), DT.BFP_BFloat8), ((hidden, ffn), DT.BFP_BFloat8),
        ((ffn, hidden), DT.BFP_BFloat4)])
    pb.begin_program("c5_decoder_layer")
    x = pb.input((1, seq, hidden), DT.BFloat16)
    anw = pb.input((hidden,), DT.BFloat16)
    wq, wk, wv, wo = (pb.input(s, DT.BFloat16) for s in ((hidden, dq), (hidden, dkv), (hidden, dkv), (dq, hidden)))
    mnw = pb.input((hidden,), DT.BFloat16)
    wg, wu, wd = pb.input((hidden, ffn), DT.BFloat16), pb.input((hidden, ffn), DT.BFloat16), pb.input((ffn, hidden), DT.BFloat16)
    qq, qk, qv, qo, qg, qu, qd = pb.load_cached(ce, "c5_decoder_const_eval_0", [wq, wk, wv, wo, wg, wu, wd], ce_outs)
    h = pb.rms_norm(x, anw, 0, eps)
    q = pb.permute(pb.reshape(pb.matmul(h, qq), (1, seq, n_q, head_dim)), (0, 2, 1, 3))
    k = pb.permute(pb.reshape(pb.matmul(h, qk), (1, seq, n_kv, head_dim)), (0, 2, 1, 3))
    v = pb.permute(pb.reshape(pb.matmul(h, qv), (1, seq, n_kv, head_dim)), (0, 2, 1, 3))
    pb.deallocate(h)
    attn = pb.sdpa(q, k, v, 0, is_causal=True)
    for t in (q, k, v):
        pb.deallocate(t)
    merged = pb.reshape(pb.permute(attn, (0, 2, 1, 3)), (1, seq, dq))
    pb.deallocate(attn)
    x1 = pb.binary(BINARY["add"], x, pb.matmul(merged, qo))
    d = _mlp(pb, x1, mnw, qg, qu, qd, eps)
    out = pb.binary(BINARY["add"], x1, d)
    pb.output(out)
    pb.end_program()
    return pb.finish()


def add_traced(pb, name, args, body, out_descs):
    """Adds the four private programs the compiler's trace hoisting emits for a traced region
    (test/ttmlir/Dialect/TTNN/trace/scenarios/single_add_no_consteval.mlir:5-45) and returns a function that emits the
    `capture_or_execute_trace` op into the program that is open when it is called.

    args: [(shape, dtype, resident[, layout])] - resident arguments live on the device (parameters, const-eval results,
    caches) and are their own slots; the others arrive on the host, row-major, and are staged into device slots.  The
    device layout is TILE unless given (positions and page tables stay row-major).
    body(pb, ids) -> [result ids] builds the traced computation on Device / Tile tensors.
    out_descs: [(shape, Layout)] of the results.

      trace_0_<name>(args..., out slots...)            body, then ttnn.copy of every result into its slot; returns nothing
      allocate_slots_trace_0_<name>(resident args...)  -> input slots (resident args pass through), output slots
      run_and_capture_trace_0_<name>(host args..., input slots..., output slots...) -> trace id
                                                       write_tensor, one eager run, capture of a second run, one replay
      execute_trace_0_<name>(trace id)                 ttnn.execute_trace
    """
    args = [(a[0], a[1], a[2], a[3] if len(a) > 3 else TL.Tile) for a in args]
    # the traced function
    pb.begin_program("trace_0_" + name, private=True)
    ids = [pb.input(shape, dt, lay) for shape, dt, _, lay in args]
    slots = [pb.input(shape, lay.dtype, lay.layout, lay.storage) for shape, lay in out_descs]
    for res, slot in zip(body(pb, ids), slots):
        pb.copy(res, slot)
    trace_fn = pb.end_program()
    # slot allocation
    pb.begin_program("allocate_slots_trace_0_" + name, private=True)
    resident = iter([pb.input(shape, dt, lay) for shape, dt, res, lay in args if res])
    for shape, dt, res, lay in args:
        pb.output(next(resident) if res else pb.empty(shape, dt, lay))
    for shape, lay in out_descs:
        pb.output(pb.empty(shape, lay.dtype, lay.layout))
    allocate = pb.end_program()
    # capture
    pb.begin_program("run_and_capture_trace_0_" + name, private=True)
    staged = [pb.input(shape, dt, TL.RowMajor, ST.Host) for shape, dt, res, _ in args if not res]
    in_slots = [pb.input(shape, dt, lay) for shape, dt, _, lay in args]
    out_slots = [pb.input(shape, lay.dtype, lay.layout, lay.storage) for shape, lay in out_descs]
    host = iter(staged)
    for (shape, dt, res, _), slot in zip(args, in_slots):
        if not res:
            pb.write_tensor(next(host), slot)
    pb.func_call(trace_fn, in_slots + out_slots, [])
    tid = pb.begin_trace_capture()
    pb.func_call(trace_fn, in_slots + out_slots, [])
    pb.end_trace_capture(tid)
    pb.execute_trace(tid)
    pb.output(tid)
    capture = pb.end_program()
    # replay
    pb.begin_program("execute_trace_0_" + name, private=True)
    tid = pb.input((), DT.UInt32, TL.RowMajor, ST.Host)
    pb.execute_trace(tid)
    execute = pb.end_program()

    def emit(pb, operands):
        return pb.capture_or_execute_trace(capture, execute, allocate, operands, out_descs)
    return emit


def traced_mlp(tokens=32, hidden=4096, ffn=14336, eps=1e-5, trace=True):
    """Decode-sized MLP block (config 4 at `tokens` rows) whose whole body is one traced region: activations arrive on the
    host, weights are device-resident parameters packed by const-eval outside the trace
    (test/ttmlir/Dialect/TTNN/trace/scenarios/matmul_multiply_consteval.mlir).  trace=False builds the same program with
    the body inline, for comparison."""
    pb = rt.ProgramBuilder()
    ce, ce_outs = _consteval_pack(pb, "traced_mlp_const_eval_0", [((hidden, ffn), DT.BFP_BFloat8), ((hidden, ffn), DT.BFP_BFloat8),
                                                                  ((ffn, hidden), DT.BFP_BFloat4)])
    out_desc = ((tokens, hidden), rt.Layout(ST.Device, TL.Tile, DT.BFloat16))
    emit = None
    if trace:
        args = [((tokens, hidden), DT.BFloat16, False), ((hidden,), DT.BFloat16, True), ((hidden, ffn), DT.BFP_BFloat8, True),
                ((hidden, ffn), DT.BFP_BFloat8, True), ((ffn, hidden), DT.BFP_BFloat4, True)]
        emit = add_traced(pb, "traced_mlp", args, lambda pb, a: [_mlp(pb, a[0], a[1], a[2], a[3], a[4], eps)], [out_desc])
    pb.begin_program("traced_mlp")
    x = pb.input((tokens, hidden), DT.BFloat16, TL.RowMajor, ST.Host)
    nw = pb.input((hidden,), DT.BFloat16)
    wg, wu, wd = pb.input((hidden, ffn), DT.BFloat16), pb.input((hidden, ffn), DT.BFloat16), pb.input((ffn, hidden), DT.BFloat16)
    qg, qu, qd = pb.load_cached(ce, "traced_mlp_const_eval_0", [wg, wu, wd], ce_outs)
    if trace:
        (y,) = emit(pb, [x, nw, qg, qu, qd])
    else:
        y = _mlp(pb, pb.to_layout(pb.to_device(x), TL.Tile), nw, qg, qu, qd, eps)
    pb.output(y)
    pb.end_program()
    return pb.finish()


def _decode_body(pb, a, users, hidden, n_q, n_kv, head_dim, eps):
    """One decode step of a Llama-style layer for `users` sequences that share a position (op mix of
    test/ttmlir/models/single_blocks_and_layers/llama_3_8b_decode_layer.mlir after RoPE / cache / attention fusing):
    a = [x, cos, sin, update_index, cur_pos, k_cache, v_cache, attn_norm_w, wq, wk, wv, wo, mlp_norm_w, wg, wu, wd]."""
    x, cos, sin, upd, cur, kc, vc, anw, wq, wk, wv, wo, mnw, wg, wu, wd = a
    h = pb.rms_norm(x, anw, 0, eps)
    # each projection is followed at once by its head split and what consumes it, in the order of the reference's layer
    # (llama_3_8b_decode_layer.mlir:51-82).  Decode-mode RoPE: cos / sin hold the row of the current position,
    # token_index = 0 (lib/Dialect/TTNN/Transforms/Fusing/RoPEFusingPattern.cpp:1143-1149)
    q = pb.rotary_embedding(pb.reshape(pb.matmul(h, wq), (1, users, n_q, head_dim)), cos, sin, token_index=0)
    k = pb.rotary_embedding(pb.reshape(pb.matmul(h, wk), (1, users, n_kv, head_dim)), cos, sin, token_index=0)
    v = pb.reshape(pb.matmul(h, wv), (1, users, n_kv, head_dim))
    pb.update_cache(vc, pb.permute(v, (0, 2, 1, 3)), upd)
    pb.update_cache(kc, pb.permute(k, (0, 2, 1, 3)), upd)
    attn = pb.sdpa_decode(q, kc, vc, cur_pos=cur, is_causal=True)
    merged = pb.reshape(attn, (users, n_q * head_dim))
    x1 = pb.binary(BINARY["add"], x, pb.matmul(merged, wo))
    d = _mlp(pb, x1, mnw, wg, wu, wd, eps)
    return pb.binary(BINARY["add"], x1, d)


def decode_layer(users=32, hidden=4096, n_q=32, n_kv=8, head_dim=128, ffn=14336, max_seq=2048, eps=1e-5, trace=False,
                 host_inputs=True):
    """Decoder layer, one new token per user, KV caches updated in place.  Inputs: x [users, hidden], cos / sin
    [1, 1, 1, head_dim] of the current position, update_index [1] and cur_pos [users] (Int32), k / v caches
    [users, n_kv, max_seq, head_dim], then the weights in bf16 (packed to block-float by const-eval).  With trace=True
    the step is one traced region: activations, rotary rows and positions are staged from the host (or, with
    host_inputs=False, are device tensors the caller updates in place), caches and weights are device resident."""
    pb = rt.ProgramBuilder()
    dq, dkv = n_q * head_dim, n_kv * head_dim
    name = "decode_layer"
    ce, ce_outs = _consteval_pack(pb, name + "_const_eval_0", [
        ((hidden, dq), DT.BFP_BFloat8), ((hidden, dkv), DT.BFP_BFloat8), ((hidden, dkv), DT.BFP_BFloat8),
        ((dq, hidden), DT.BFP_BFloat8), ((hidden, ffn), DT.BFP_BFloat8), ((hidden, ffn), DT.BFP_BFloat8),
        ((ffn, hidden), DT.BFP_BFloat4)])
    cache_shape = (users, n_kv, max_seq, head_dim)
    on_dev = not host_inputs
    step = [((users, hidden), DT.BFloat16, on_dev), ((1, 1, 1, head_dim), DT.BFloat16, on_dev), ((1, 1, 1, head_dim), DT.BFloat16, on_dev),
            ((1,), DT.Int32, on_dev, TL.RowMajor), ((users,), DT.Int32, on_dev, TL.RowMajor),
            (cache_shape, DT.BFloat16, True), (cache_shape, DT.BFloat16, True)]
    wshapes = [(hidden,), (hidden, dq), (hidden, dkv), (hidden, dkv), (dq, hidden), (hidden,), (hidden, ffn), (hidden, ffn), (ffn, hidden)]
    wdtypes = [DT.BFloat16, DT.BFP_BFloat8, DT.BFP_BFloat8, DT.BFP_BFloat8, DT.BFP_BFloat8, DT.BFloat16, DT.BFP_BFloat8, DT.BFP_BFloat8,
               DT.BFP_BFloat4]
    out_desc = ((users, hidden), rt.Layout(ST.Device, TL.Tile, DT.BFloat16))
    body = lambda pb, a: [_decode_body(pb, a, users, hidden, n_q, n_kv, head_dim, eps)]
    emit = None
    if trace:
        emit = add_traced(pb, name, step + [(s, d, True) for s, d in zip(wshapes, wdtypes)], body, [out_desc])
    pb.begin_program(name)
    ins = []
    for a in step:
        shape, dt, resident = a[0], a[1], a[2]
        lay = a[3] if len(a) > 3 else TL.Tile
        if trace and not resident:
            ins.append(pb.input(shape, dt, TL.RowMajor, ST.Host))
        else:
            ins.append(pb.input(shape, dt, lay))
    raw = [pb.input(s, DT.BFloat16) for s in wshapes]
    packed = pb.load_cached(ce, name + "_const_eval_0", [raw[1], raw[2], raw[3], raw[4], raw[6], raw[7], raw[8]], ce_outs)
    weights = [raw[0], packed[0], packed[1], packed[2], packed[3], raw[5], packed[4], packed[5], packed[6]]
    out = emit(pb, ins + weights)[0] if trace else body(pb, ins + weights)[0]
    pb.output(out)
    pb.end_program()
    return pb.finish()
