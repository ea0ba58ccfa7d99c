"""GPU parity of the bandwidth kernels, data movement and attention against the CPU oracle on
identical seeded inputs.  Tolerances: fp32 tensors -- values agree to 1e-5 relative (different
transcendental implementations); bf16 tensors -- at most one bf16 ulp of the result (2^-8
relative); PCC >= 0.99 everywhere (north star), asserted much tighter."""
import numpy as np
import pytest
import torch

from ttmlir_amd import datagen
from test_gpu_linear import tilize_dev, untilize_dev

pytestmark = pytest.mark.gpu


def bf16_ulps(got, want):
    """|got - want| in units of the bf16 spacing at |want| (both f32 arrays holding bf16 values)."""
    _, e = np.frexp(np.clip(np.abs(want), 2.0 ** -126, 3e38))
    with np.errstate(invalid="ignore"):
        d = np.where(got == want, 0.0, np.abs(got - want))          # equal infinities count as exact
    return d / np.ldexp(1.0, e - 8)


UNARY = ["abs", "ceil", "cos", "floor", "gelu", "isfinite", "logical_not", "neg", "relu", "sqrt", "rsqrt", "sigmoid",
         "sin", "reciprocal", "sign", "tanh", "atan", "exp", "erf", "erfc", "log", "expm1", "relu6", "silu", "leaky_relu",
         "hardsigmoid", "mish", "acos", "asin", "asinh", "cbrt", "log1p"]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_unary(hip, dev, orc, dtype):
    x = datagen.randn((70, 33), seed=1, std=2.0)
    x[0, :4] = torch.tensor([0.0, -0.0, 1.0, -1.0])
    for name in UNARY:
        xi = x.abs() + 0.01 if name in ("sqrt", "rsqrt", "log", "log1p") else x
        if name in ("acos", "asin"):
            xi = torch.tanh(x)
        if dtype == "bf16":
            xi = xi.to(torch.bfloat16)
        xd = xi.to(dev)
        out = torch.empty_like(xd)
        hip.call("ttm_eltwise_unary", orc.UNARY[name], hip.ptr(xd), hip.ptr(out), hip.BF16 if dtype == "bf16" else hip.F32,
                 hip.ROW_MAJOR, 1, 70, 33, 0.1, hip.current_stream())
        torch.cuda.synchronize()
        want = orc.unary(name, xi.float().numpy(), 0.1)
        got = out.float().cpu().numpy()
        if dtype == "f32":
            assert np.allclose(got, want, rtol=1e-5, atol=1e-6), name
        else:
            assert np.max(bf16_ulps(got, orc.round_bf16(want))) <= 1.0, name


@pytest.mark.parametrize("layout", ["tile", "row_major"])
@pytest.mark.parametrize("ashape,bshape", [((64, 96), (64, 96)), ((2, 3, 40, 50), (2, 3, 40, 50)), ((64, 96), (1, 96)),
                                           ((2, 64, 96), (64, 1)), ((2, 1, 33, 70), (1, 3, 1, 70)), ((4, 32, 32), (1,)),
                                           ((1, 128), (5, 128, 1)), ((2, 40, 64), (1, 64)), ((3, 70, 96), (3, 1, 96)),
                                           ((2, 2, 33, 128), (2, 1, 33, 1))])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_binary_broadcast(hip, dev, orc, layout, ashape, bshape, dtype):
    """Same-shape, row-vector, column-vector, scalar and batch broadcasting in both layouts and dtypes: the flat kernel, the
    16-byte-chunk kernel (rows of whole chunks, ragged row counts included) and the element-wise one (ragged columns)."""
    a = datagen.randn(ashape, seed=2, dtype=dtype)
    b = datagen.randn(bshape, seed=3, dtype=dtype) + 3.0
    oshape = tuple(np.broadcast_shapes(ashape, bshape))
    rank = len(oshape)
    pad = lambda s: np.array((1,) * (rank - len(s)) + tuple(s), dtype=np.int64)
    tiled = layout == "tile"
    r2 = lambda t: t.reshape((1,) * (2 - t.dim()) + tuple(t.shape)) if t.dim() < 2 else t
    for name in ("add", "multiply", "subtract", "divide", "gt"):
        if tiled:
            ad, bd = tilize_dev(hip, r2(a), dev), tilize_dev(hip, r2(b), dev)
            Rp, Cp = (oshape[-2] + 31) // 32 * 32, (oshape[-1] + 31) // 32 * 32
            od = torch.full((int(np.prod(oshape[:-2], dtype=np.int64)) * Rp * Cp,), float("nan"), dtype=dtype, device=dev)
        else:
            ad, bd = a.to(dev), b.to(dev)
            od = torch.empty(oshape, dtype=dtype, device=dev)
        sa, sb, so = pad(ashape), pad(bshape), pad(oshape)          # keep the shape arrays alive over the call
        hip.call("ttm_eltwise_binary", orc.BINARY[name], hip.ptr(ad), sa.ctypes.data, hip.ptr(bd),
                 sb.ctypes.data, hip.ptr(od), so.ctypes.data, rank, hip.BF16 if dtype == torch.bfloat16 else hip.F32,
                 hip.TILE if tiled else hip.ROW_MAJOR, hip.current_stream())
        res = untilize_dev(hip, od, oshape, dev) if tiled else od
        torch.cuda.synchronize()
        want = orc.binary(name, a.float().numpy(), b.float().numpy())
        if dtype == torch.bfloat16:
            want = orc.round_bf16(want)
        assert np.array_equal(res.float().cpu().numpy(), want), name   # one rounding of an exact f32 op: bit exact
        if tiled:  # padding of the tiled result is zero
            full = od.float().cpu().numpy()
            assert np.count_nonzero(full) == np.count_nonzero(want)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(2, 40, 50), (3, 70, 64), (1, 32, 33), (2, 1, 1)])
def test_unary_keeps_tile_padding_zero(hip, dev, orc, shape, dtype):
    """Ops with f(0) != 0 on tile tensors with ragged rows, ragged columns or both: the padding stays zero."""
    x = datagen.randn(shape, seed=21, dtype=dtype)
    xt = tilize_dev(hip, x, dev)
    for name in ("exp", "reciprocal", "gelu"):
        out = torch.full_like(xt, float("nan"))
        hip.call("ttm_eltwise_unary", orc.UNARY[name], hip.ptr(xt), hip.ptr(out), hip.BF16 if dtype == torch.bfloat16 else hip.F32, hip.TILE,
                 shape[0], shape[1], shape[2], 0.0, hip.current_stream())
        torch.cuda.synchronize()
        want = orc.unary(name, x.float().numpy())
        if dtype == torch.bfloat16:
            want = orc.round_bf16(want)
        full = out.float().cpu().numpy()
        wt = orc.tilize(want)
        assert np.array_equal(full == 0, wt == 0)                               # padding (and only padding) is zero
        got = untilize_dev(hip, out, x.shape, dev).float().cpu().numpy()
        if dtype == torch.bfloat16:
            assert np.max(bf16_ulps(got, want)) <= 1.0
        else:
            assert np.allclose(got, want, rtol=1e-5, atol=1e-6)


def test_typecast(hip, dev, orc):
    x = datagen.randn((1000,), seed=4, std=300.0)
    x[:6] = torch.tensor([0.0, -0.0, 1e10, -1e10, 65535.4, -7.9])
    xd = x.to(dev)
    s = hip.current_stream()
    out = torch.empty(1000, dtype=torch.bfloat16, device=dev)
    hip.call("ttm_typecast", hip.ptr(xd), hip.F32, hip.ptr(out), hip.BF16, 1000, s)
    assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), orc.f32_to_bf16(x.numpy()))
    back = torch.empty(1000, dtype=torch.float32, device=dev)
    hip.call("ttm_typecast", hip.ptr(out), hip.BF16, hip.ptr(back), hip.F32, 1000, s)
    assert torch.equal(back.cpu(), out.float().cpu())
    i32 = torch.empty(1000, dtype=torch.int32, device=dev)
    hip.call("ttm_typecast", hip.ptr(xd), hip.F32, hip.ptr(i32), hip.I32, 1000, s)
    want = np.clip(np.trunc(x.double().numpy()), -2 ** 31, 2 ** 31 - 1).astype(np.int64)
    assert np.array_equal(i32.cpu().numpy().astype(np.int64), want)
    u8 = torch.empty(1000, dtype=torch.uint8, device=dev)
    hip.call("ttm_typecast", hip.ptr(i32), hip.I32, hip.ptr(u8), hip.U8, 1000, s)
    assert np.array_equal(u8.cpu().numpy().astype(np.int64), np.clip(want, 0, 255))   # saturating narrowing
    f16 = torch.empty(1000, dtype=torch.float16, device=dev)
    hip.call("ttm_typecast", hip.ptr(out), hip.BF16, hip.ptr(f16), hip.F16, 1000, s)
    torch.cuda.synchronize()
    sel = np.abs(out.float().cpu().numpy()) < 65504
    assert np.array_equal(f16.view(torch.int16).cpu().numpy().view(np.uint16)[sel],
                          orc.bf16_to_f16(out.view(torch.int16).cpu().numpy().view(np.uint16))[sel])


@pytest.fixture(params=[0, 1, 2, 3], ids=["auto", "resident", "band", "row"])
def rowwise_variant(request, hip):
    """Every row-wise kernel on every shape: 0 = by size, 1 = eight rows per workgroup parked in LDS (or the re-reading
    kernel), 2 = four rows per workgroup in registers, 3 = one row per workgroup."""
    hip.set_option("rowwise_variant", request.param)
    yield request.param
    hip.set_option("rowwise_variant", 0)


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("shape,wl,bias", [((512, 4096), "tile", False), ((64, 96), "tile", True), ((3, 40, 70), "rm", True),
                                           ((1, 33), "tile", False), ((2, 2, 32, 256), "rm", False), ((2048, 1024), "tile", True),
                                           ((40, 8192), "rm", False), ((64, 16384), "tile", True), ((33, 6000), "rm", True),
                                           ((40, 8200), "tile", True), ((33, 16500), "rm", True)])   # few very wide rows: two steps over column slices
def test_rms_norm(hip, dev, orc, dtype, shape, wl, bias, rowwise_variant):
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float32
    x = datagen.randn(shape, seed=5, dtype=tdt)
    C = shape[-1]
    w = (1.0 + 0.02 * datagen.randn((C,), seed=6)).to(tdt)
    b = datagen.randn((C,), seed=7, std=0.1).to(tdt) if bias else None
    xt = tilize_dev(hip, x, dev)
    vec = lambda v: tilize_dev(hip, v.reshape(1, -1), dev) if wl == "tile" else v.to(dev)
    wd, bd = vec(w), (vec(b) if bias else None)
    out = torch.full_like(xt, float("nan"))
    batch, R = int(np.prod(shape[:-2], dtype=np.int64)), shape[-2]
    lay = hip.TILE if wl == "tile" else hip.ROW_MAJOR
    hip.call("ttm_rms_norm", hip.ptr(xt), hip.ptr(wd), lay, hip.ptr(bd) if bias else None, lay, hip.ptr(out),
             hip.BF16 if dtype == "bf16" else hip.F32, batch, R, C, 1e-5, hip.current_stream())
    res = untilize_dev(hip, out, shape, dev)
    torch.cuda.synchronize()
    want = orc.rms_norm(x.float().numpy(), w.float().numpy(), None if b is None else b.float().numpy(), 1e-5)
    got = res.float().cpu().numpy()
    if dtype == "f32":
        assert np.allclose(got, want, rtol=2e-5, atol=1e-6)
    else:
        # one bf16 spacing at the size of the terms: where x / rms * w and the bias cancel, the fp32 difference of two O(1)
        # numbers (fused or separately rounded) is all there is, and a spacing of the tiny result would be finer than it
        wr = orc.round_bf16(want)
        scale = np.abs(wr) if b is None else np.maximum(np.abs(wr), np.abs(b.float().numpy()))
        assert np.all(np.abs(got - wr) <= np.exp2(np.floor(np.log2(np.maximum(scale, 2.0 ** -120))) - 7))
    assert np.all(np.isfinite(out.float().cpu().numpy()))          # padding written as zeros, not left NaN


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("shape", [(64, 96), (2, 3, 40, 70), (1, 2048), (32, 2048), (1100, 300), (3, 33, 4100), (64, 8192), (33, 12000), (40, 8200), (2, 33, 16500), (3, 50000)])
def test_softmax_and_reduce_lastdim(hip, dev, orc, dtype, shape, rowwise_variant):
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float32
    hdt = hip.BF16 if dtype == "bf16" else hip.F32
    x = datagen.randn(shape, seed=8, std=3.0, dtype=tdt)
    xt = tilize_dev(hip, x, dev)
    batch, R, C = int(np.prod(shape[:-2], dtype=np.int64)), shape[-2], shape[-1]
    out = torch.full_like(xt, float("nan"))
    hip.call("ttm_softmax_lastdim", hip.ptr(xt), hip.ptr(out), hdt, batch, R, C, hip.current_stream())
    res = untilize_dev(hip, out, shape, dev).float().cpu().numpy()
    want = orc.softmax(x.float().numpy(), -1)
    if dtype == "f32":
        # the oracle sums a row in fp32 one element after another: over thousands of columns that drifts further from the
        # exact value than the kernels' tree sums do, so both are held against the float64 result, each to its own bound
        x64 = x.double().numpy()
        ref = np.exp(x64 - x64.max(-1, keepdims=True))
        ref /= ref.sum(-1, keepdims=True)
        assert np.allclose(want, ref, rtol=max(2e-5, 1.2e-7 * C), atol=1e-7)
        assert np.allclose(res, ref, rtol=2e-5, atol=1e-7)
    else:
        assert np.max(bf16_ulps(res, orc.round_bf16(want))) <= 1.0
    Rp = (R + 31) // 32 * 32
    for op in ("sum", "mean", "max", "min"):
        o = torch.full((batch * Rp * 32,), float("nan"), dtype=tdt, device=dev)
        hip.call("ttm_reduce_lastdim", orc.REDUCE[op], hip.ptr(xt), hip.ptr(o), hdt, batch, R, C, hip.current_stream())
        got = untilize_dev(hip, o, tuple(shape[:-1]) + (1,), dev).float().cpu().numpy()
        w = orc.reduce(op, x.float().numpy(), -1, keepdim=True)
        if dtype == "f32":
            # fp32 sums in another order than the oracle's: both within n eps of the exact sum of magnitudes (max / min: exact)
            mag = np.abs(x.float().numpy()).sum(-1, keepdims=True) / (C if op == "mean" else 1)
            atol = 0.0 if op in ("max", "min") else 2.0 ** -22 * mag
            assert np.all(np.abs(got - w) <= 1e-6 * np.abs(w) + atol), op
        else:
            assert np.max(bf16_ulps(got, orc.round_bf16(w))) <= 1.0, op
        assert np.all(np.isfinite(o.float().cpu().numpy()))

def _same_specials(got, want, what):
    """NaN in the same places, the same infinities, and equal values elsewhere up to `tol` bf16 / fp32 handling by the caller."""
    assert np.array_equal(np.isnan(got), np.isnan(want)), what + ": NaN in other places than in the oracle's result"
    assert np.array_equal(np.isposinf(got), np.isposinf(want)) and np.array_equal(np.isneginf(got), np.isneginf(want)), what + ": infinities differ"


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("shape", [(64, 96), (2, 40, 70), (32, 2048), (33, 4100), (40, 8200), (3, 50000)])
def test_rowwise_ops_on_rows_with_nan_inf_and_negative_zero(hip, dev, orc, dtype, shape, rowwise_variant):
    """NaN, +-Inf and -0.0 through sum / mean / max / min, softmax and RMSNorm in every row-wise kernel: max and min return
    NaN for a row that holds one (tosa.reduce_max / reduce_min propagate, lib/Conversion/TTIRToLinalg/Reduction.cpp:133-136;
    torch.max / torch.min of the goldens, tools/golden/mapping.py:5189-5220, 2815-2856), an infinity wins over finite values,
    a row of -0.0 keeps its sign.  Rows without special values are checked as in the ordinary tests."""
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float32
    hdt = hip.BF16 if dtype == "bf16" else hip.F32
    x = datagen.randn(shape, seed=88, std=2.0, dtype=tdt)
    R, C = shape[-2], shape[-1]
    xf = x.reshape(-1, C)
    nan, inf = float("nan"), float("inf")
    rows = xf.shape[0]
    special = {0: [(0, nan)], 1: [(C - 1, nan)], 2: [(C // 2, inf)], 3: [(1, -inf)], 4: [(3, inf), (C - 2, -inf)],
               5: [(2, nan), (5, inf)], 6: [(C // 3, -inf), (C // 3 + 1, nan)], 9: [(C - 1, inf)], 10: [(0, -inf), (C - 1, -inf)]}
    for r, cells in special.items():
        if r < rows:
            for c, v in cells:
                xf[r, c] = v
    if rows > 7:
        xf[7, :] = -0.0
    if rows > 8:
        xf[8, :] = -inf
    if rows > 11:
        xf[11, :] = 0.0
        xf[11, C // 2] = -0.0
    xt = tilize_dev(hip, x, dev)
    batch = int(np.prod(shape[:-2], dtype=np.int64))
    xn = x.float().numpy()
    Rp = (R + 31) // 32 * 32
    for op in ("sum", "mean", "max", "min"):
        o = torch.full((batch * Rp * 32,), 7.0, dtype=tdt, device=dev)
        hip.call("ttm_reduce_lastdim", orc.REDUCE[op], hip.ptr(xt), hip.ptr(o), hdt, batch, R, C, hip.current_stream())
        got = untilize_dev(hip, o, tuple(shape[:-1]) + (1,), dev).float().cpu().numpy()
        with np.errstate(invalid="ignore", over="ignore"):
            want = orc.reduce(op, xn, -1, keepdim=True)
        want = orc.round_bf16(want) if dtype == "bf16" else want
        _same_specials(got, want, op)
        fin = np.isfinite(want)
        if op in ("max", "min"):
            assert np.array_equal(got[fin], want[fin]), op            # exact, zeros of either sign equal
            if rows > 7:
                assert np.signbit(got.reshape(-1)[7]), op + " of a row of -0.0"
        elif dtype == "f32":
            mag = np.abs(np.where(np.isfinite(xn), xn, 0)).sum(-1, keepdims=True) / (C if op == "mean" else 1)
            assert np.all(np.abs(got[fin] - want[fin]) <= 1e-6 * np.abs(want[fin]) + 2.0 ** -22 * mag[fin]), op
        else:
            assert not fin.any() or np.max(bf16_ulps(got[fin], want[fin])) <= 1.0, op
    out = torch.full_like(xt, 7.0)
    hip.call("ttm_softmax_lastdim", hip.ptr(xt), hip.ptr(out), hdt, batch, R, C, hip.current_stream())
    res = untilize_dev(hip, out, shape, dev).float().cpu().numpy()
    with np.errstate(invalid="ignore", over="ignore"):
        want = orc.softmax(xn, -1)
    want = orc.round_bf16(want) if dtype == "bf16" else want
    _same_specials(res, want, "softmax")
    fin = np.isfinite(want)
    if dtype == "f32":
        assert np.allclose(res[fin], want[fin], rtol=max(2e-5, 1.2e-7 * C), atol=1e-7)
    else:
        assert not fin.any() or np.max(bf16_ulps(res[fin], want[fin])) <= 1.0
    w = (1.0 + 0.02 * datagen.randn((C,), seed=6)).to(tdt)
    wd = w.to(dev)
    out = torch.full_like(xt, 7.0)
    hip.call("ttm_rms_norm", hip.ptr(xt), hip.ptr(wd), hip.ROW_MAJOR, None, hip.ROW_MAJOR, hip.ptr(out), hdt, batch, R, C, 1e-5,
             hip.current_stream())
    res = untilize_dev(hip, out, shape, dev).float().cpu().numpy()
    with np.errstate(invalid="ignore", over="ignore"):
        want = orc.rms_norm(xn, w.float().numpy(), None, 1e-5)
    want = orc.round_bf16(want) if dtype == "bf16" else want
    _same_specials(res, want, "rms_norm")
    fin = np.isfinite(want)
    if dtype == "f32":
        assert np.allclose(res[fin], want[fin], rtol=2e-5, atol=1e-6)
    else:
        assert not fin.any() or np.max(bf16_ulps(res[fin], want[fin])) <= 1.0
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(64, 96), (3, 128, 32), (2, 2, 32, 160), (1024, 2048)])
@pytest.mark.parametrize("dst_order", [False, True])
def test_tile_transpose_of_whole_tiles(hip, dev, dtype, shape, dst_order):
    """The transpose of the last two dims between tile-order tensors of whole tiles (the dedicated kernel): the view written
    in destination order, as the runtime does, and in source order; batched; against torch.transpose."""
    x = datagen.randn(shape, seed=12, dtype=dtype)
    xt = tilize_dev(hip, x, dev)
    tshape = tuple(shape[:-2]) + (shape[-1], shape[-2])
    xs, ts = strides(shape), strides(tshape)
    if dst_order:   # view dims run over the destination's shape; the source is read with swapped strides
        out = view_copy(hip, dev, xt, shape, True, tshape, True, tshape, xs[:-2] + [xs[-1], xs[-2]], ts)
    else:           # view dims run over the source's shape; the destination is written with swapped strides
        out = view_copy(hip, dev, xt, shape, True, tshape, True, shape, xs, ts[:-2] + [ts[-1], ts[-2]])
    torch.cuda.synchronize()
    assert torch.equal(untilize_dev(hip, out, tshape, dev).cpu(), x.transpose(-1, -2).contiguous())


def view_copy(hip, dev, src, src_shape, src_tiled, dst_shape, dst_tiled, extent, sstride, dstride, sbase=0, dbase=0,
              dst=None):
    r2 = lambda s: (1,) * (2 - len(s)) + tuple(s) if len(s) < 2 else tuple(s)
    ss, ds = r2(src_shape), r2(dst_shape)
    if dst is None:
        n = int(np.prod(ds[:-2], dtype=np.int64)) * ((ds[-2] + 31) // 32 * 32) * ((ds[-1] + 31) // 32 * 32) if dst_tiled \
            else int(np.prod(ds, dtype=np.int64))
        dst = torch.zeros(n, dtype=src.dtype, device=dev)
    e, s1, s2 = (np.array(v, dtype=np.int64) for v in (extent, sstride, dstride))
    hip.call("ttm_copy_view", hip.ptr(src), ss[-2], ss[-1], hip.TILE if src_tiled else hip.ROW_MAJOR, hip.ptr(dst),
             ds[-2], ds[-1], hip.TILE if dst_tiled else hip.ROW_MAJOR, src.element_size(), len(extent),
             e.ctypes.data, s1.ctypes.data, sbase, s2.ctypes.data, dbase, hip.current_stream())
    return dst


def strides(shape):
    s, acc = [], 1
    for d in reversed(shape):
        s.insert(0, acc)
        acc *= d
    return s


def test_copy_view_reshape_permute_slice_concat(hip, dev, orc):
    x = datagen.randn((2, 48, 64), seed=9, dtype=torch.bfloat16)
    xt = tilize_dev(hip, x, dev)
    # reshape [2,48,64] -> [2,48,4,16] -> permute (0,2,1,3) -> [2,4,48,16], tiled in and out
    oshape = (2, 4, 48, 16)
    in4 = strides((2, 48, 4, 16))
    out = view_copy(hip, dev, xt, (2, 48, 64), True, oshape, True, oshape, [in4[0], in4[2], in4[1], in4[3]], strides(oshape))
    got = untilize_dev(hip, out, oshape, dev).cpu()
    assert torch.equal(got, x.reshape(2, 48, 4, 16).permute(0, 2, 1, 3))
    # slice [:, 8:40:2, 16:48] to row-major
    sl = x[:, 8:40:2, 16:48]
    i3 = strides((2, 48, 64))
    out = view_copy(hip, dev, xt, (2, 48, 64), True, sl.shape, False, sl.shape, [i3[0], 2 * i3[1], i3[2]],
                    strides(sl.shape), sbase=8 * 64 + 16)
    assert torch.equal(out.reshape(sl.shape).cpu(), sl)
    # concat along dim 1 of two tiled tensors into a tiled [2, 96, 64]
    y = datagen.randn((2, 48, 64), seed=10, dtype=torch.bfloat16)
    yt = tilize_dev(hip, y, dev)
    cshape = (2, 96, 64)
    dst = view_copy(hip, dev, xt, x.shape, True, cshape, True, x.shape, strides(x.shape), strides(cshape))
    dst = view_copy(hip, dev, yt, y.shape, True, cshape, True, y.shape, strides(y.shape), strides(cshape), dbase=48 * 64, dst=dst)
    assert torch.equal(untilize_dev(hip, dst, cshape, dev).cpu(), torch.cat([x, y], dim=1))
    # repeat_interleave(3, dim=0): view [2,3,48,64] with source stride 0 on the repeat dim
    rshape = (6, 48, 64)
    dst = view_copy(hip, dev, xt, x.shape, True, rshape, True, (2, 3, 48, 64), [i3[0], 0, i3[1], i3[2]],
                    strides((2, 3, 48, 64)))
    assert torch.equal(untilize_dev(hip, dst, rshape, dev).cpu(), x.repeat_interleave(3, dim=0))
    # transpose of the last two dims on fp32, ragged
    z = datagen.randn((3, 40, 50), seed=11)
    zt = tilize_dev(hip, z, dev)
    tshape = (3, 50, 40)
    zs = strides(z.shape)
    dst = view_copy(hip, dev, zt, z.shape, True, tshape, True, tshape, [zs[0], zs[2], zs[1]], strides(tshape))
    torch.cuda.synchronize()
    assert torch.equal(untilize_dev(hip, dst, tshape, dev).cpu(), z.transpose(1, 2))
    assert np.array_equal(dst.cpu().numpy(), orc.tilize(z.transpose(1, 2).contiguous().numpy()))   # padding stays zero


@pytest.mark.parametrize("batch", [4, 5])
def test_copy_view_index_width_boundary(hip, dev, batch):
    """The copy kernels index with 32 bits when every logical and padded offset stays below 2^29 elements and with 64
    bits otherwise: [4, 8192, 16384] bf16 (2^29 elements, 1 GiB) is the largest narrow case, [5, ...] the first wide one.
    A head-split permute of both, tile layout in and out, compared with torch on the device."""
    R, C, H = 8192, 16384, 8
    g = torch.Generator(device="cpu").manual_seed(3)
    base = torch.randint(-30000, 30000, (R, C // 64), generator=g, dtype=torch.int16)
    x = base.repeat(1, 64).view(torch.bfloat16).to(dev).unsqueeze(0).repeat(batch, 1, 1)      # [batch, R, C], cheap to make
    x += torch.arange(batch, device=dev, dtype=torch.bfloat16).view(batch, 1, 1)              # batches differ
    xt = torch.empty(batch * R * C, dtype=torch.bfloat16, device=dev)
    hip.call("ttm_tilize", hip.ptr(x), hip.ptr(xt), batch, R, C, 2, hip.current_stream())
    oshape = (batch, H, R, C // H)
    in4 = strides((batch, R, H, C // H))
    out = view_copy(hip, dev, xt, (batch, R, C), True, oshape, True, oshape, [in4[0], in4[2], in4[1], in4[3]], strides(oshape))
    got = torch.empty(oshape, dtype=torch.bfloat16, device=dev)
    hip.call("ttm_untilize", hip.ptr(out), hip.ptr(got), batch * H, R, C // H, 2, hip.current_stream())
    torch.cuda.synchronize()
    want = x.view(batch, R, H, C // H).permute(0, 2, 1, 3)
    assert torch.equal(got.view(torch.int16), want.contiguous().view(torch.int16))


@pytest.mark.parametrize("index,limit", [(0, 16), (15, 16), (16, 16), (-3, 16)])
@pytest.mark.parametrize("elem", ["bf16", "f32"])
def test_copy_view_at_positions_the_destination_from_device_memory(hip, dev, elem, index, limit):
    """ttm_copy_view_at: destination base + *index * index_stride with *index read by the kernel; outside [0, limit)
    nothing is written.  A [3, 40] block goes to row block `index` of a [limit * 3, 40] row-major tensor, from a tiled
    source read through a transposing view."""
    dt = torch.bfloat16 if elem == "bf16" else torch.float32
    src = datagen.randn((40, 3), seed=12, dtype=dt)
    st = tilize_dev(hip, src, dev)
    dst0 = datagen.randn((limit * 3, 40), seed=13, dtype=dt)
    dst = dst0.clone().to(dev)
    idx = torch.tensor([index], dtype=torch.int32, device=dev)
    e, s1, s2 = (np.array(v, dtype=np.int64) for v in ([3, 40], [1, 3], [40, 1]))
    hip.call("ttm_copy_view_at", hip.ptr(st), 40, 3, hip.TILE, hip.ptr(dst), limit * 3, 40, hip.ROW_MAJOR, src.element_size(), 2,
             e.ctypes.data, s1.ctypes.data, 0, s2.ctypes.data, 0, hip.ptr(idx), 3 * 40, limit, hip.current_stream())
    torch.cuda.synchronize()
    want = dst0.clone()
    if 0 <= index < limit:
        want[3 * index:3 * index + 3] = src.t()
    assert torch.equal(dst.cpu(), want)
    with pytest.raises(hip.TTMError, match="null index"):
        hip.call("ttm_copy_view_at", hip.ptr(st), 40, 3, hip.TILE, hip.ptr(dst), limit * 3, 40, hip.ROW_MAJOR, src.element_size(), 2,
                 e.ctypes.data, s1.ctypes.data, 0, s2.ctypes.data, 0, None, 3 * 40, limit, hip.current_stream())


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal,mask", [
    (1, 4, 2, 128, 128, 64, True, None), (2, 2, 2, 96, 160, 128, False, None), (1, 8, 2, 256, 256, 128, True, None),
    (1, 2, 1, 70, 70, 32, True, None), (1, 2, 2, 64, 100, 64, False, "b1"), (2, 2, 1, 64, 64, 64, False, "bh"),
    (1, 1, 1, 40, 300, 256, False, None),
    # odd and ragged key-tile counts for the 64-keys-per-pass kernel, masks on its second half, causal with Sq != Sk
    (1, 2, 2, 160, 96, 128, False, None), (1, 4, 1, 33, 33, 128, True, None), (1, 2, 2, 96, 224, 64, False, "bh"),
    (2, 4, 4, 130, 190, 128, False, "b1"), (1, 4, 2, 192, 320, 128, True, None), (1, 2, 1, 320, 192, 32, True, None),
    (1, 8, 2, 1024, 1024, 128, True, None),
    # few query blocks against many keys: the keys of a query block shared among workgroups and merged by a second kernel
    # (variant 5 keeps them in one workgroup); ragged key counts, masks, a causal chunk, shares without any visible key
    (1, 8, 2, 128, 2048, 128, False, None), (1, 4, 2, 100, 1500, 64, False, "bh"), (2, 2, 2, 64, 1100, 128, False, "b1"),
    (1, 4, 4, 128, 1024, 128, True, None), (1, 2, 1, 40, 4096, 32, False, None)])
@pytest.mark.parametrize("variant", [0, 1, 3, 4, 5, 6, 7, 8])   # automatic, 32-key kernel, eight-wavefront kernel forced / forbidden, no key shares, no pipeline, four- / eight-wavefront pipeline
def test_sdpa(hip, dev, orc, B, Hq, Hkv, Sq, Sk, D, causal, mask, variant):
    if variant == 1 and Sq * Sk >= 512 * 512:
        pytest.skip("the 32-key kernel is covered by the small shapes")
    hip.set_option("sdpa_variant", variant)
    import oracle.metrics as metrics
    q = datagen.randn((B, Hq, Sq, D), seed=12, dtype=torch.bfloat16)
    k = datagen.randn((B, Hkv, Sk, D), seed=13, dtype=torch.bfloat16)
    v = datagen.randn((B, Hkv, Sk, D), seed=14, dtype=torch.bfloat16)
    m = None
    if mask:
        m = datagen.randn((B, 1 if mask == "b1" else Hq, Sq, Sk), seed=15, dtype=torch.bfloat16)
    qt, kt, vt = (tilize_dev(hip, t, dev) for t in (q, k, v))
    mt = tilize_dev(hip, m, dev) if m is not None else None
    out = torch.full_like(qt, float("nan"))
    try:
        hip.call("ttm_sdpa", hip.ptr(qt), hip.ptr(kt), hip.ptr(vt), hip.ptr(mt) if mt is not None else None,
                 m.shape[1] if m is not None else 1, hip.ptr(out), hip.BF16, B, Hq, Hkv, Sq, Sk, D, int(causal), 0.0,
                 hip.current_stream())
    finally:
        hip.set_option("sdpa_variant", 0)
    res = untilize_dev(hip, out, q.shape, dev).float().cpu().numpy()
    torch.cuda.synchronize()
    want = orc.sdpa(q.float().numpy(), k.float().numpy(), v.float().numpy(), None if m is None else m.float().numpy(),
                    is_causal=causal)
    assert np.all(np.isfinite(out.float().cpu().numpy()))
    # probabilities are rounded to bf16 before P.V (relative 2^-9 each) and the output once more
    assert np.max(np.abs(res - want)) <= 2.0 ** -6
    assert metrics.get_pcc(want, res) >= 0.9999


def test_sdpa_config5_shape(hip, dev, orc):
    """The attention of config 5 alone: 32 query / 8 kv heads, 2048 x 2048 causal, head dim 128 (one workgroup per CU, the
    eight-wavefront kernel), every output against the oracle."""
    import oracle.metrics as metrics
    B, Hq, Hkv, S, D = 1, 32, 8, 2048, 128
    q = datagen.randn((B, Hq, S, D), seed=112, dtype=torch.bfloat16)
    k = datagen.randn((B, Hkv, S, D), seed=113, dtype=torch.bfloat16)
    v = datagen.randn((B, Hkv, S, D), seed=114, dtype=torch.bfloat16)
    qt, kt, vt = (tilize_dev(hip, t, dev) for t in (q, k, v))
    out = torch.full_like(qt, float("nan"))
    hip.call("ttm_sdpa", hip.ptr(qt), hip.ptr(kt), hip.ptr(vt), None, 1, hip.ptr(out), hip.BF16, B, Hq, Hkv, S, S, D, 1, 0.0,
             hip.current_stream())
    res = untilize_dev(hip, out, q.shape, dev).float().cpu().numpy()
    orc.set_threads(orc.max_threads())
    try:
        want = orc.sdpa(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, is_causal=True)
    finally:
        orc.set_threads(1)
    assert np.all(np.isfinite(res))
    # probabilities are rounded to bf16 before P.V (relative 2^-9 each) and the output once more
    assert np.max(np.abs(res - want)) <= 2.0 ** -6
    assert metrics.get_pcc(want, res) >= 0.9999
    # the first query of every head sees one key: the output is that value row, exactly
    assert np.array_equal(res[0, :, 0, :], np.repeat(v.float().numpy()[0, :, 0, :], Hq // Hkv, axis=0))


def test_sdpa_several_sequences_four_wavefront_form(hip, dev, orc):
    """Three sequences of 1024 tokens (32 query / 8 kv heads, head dim 128, causal): three query blocks per CU, which the
    automatic choice gives to the four-wavefront pipelined kernel (two workgroups per CU, 32 keys per pass).  Every output
    against the oracle, and the forced eight-wavefront form beside it."""
    import oracle.metrics as metrics
    B, Hq, Hkv, S, D = 3, 32, 8, 1024, 128
    q = datagen.randn((B, Hq, S, D), seed=115, dtype=torch.bfloat16)
    k = datagen.randn((B, Hkv, S, D), seed=116, dtype=torch.bfloat16)
    v = datagen.randn((B, Hkv, S, D), seed=117, dtype=torch.bfloat16)
    qt, kt, vt = (tilize_dev(hip, t, dev) for t in (q, k, v))
    res = {}
    try:
        for variant in (0, 7, 8):
            hip.set_option("sdpa_variant", variant)
            out = torch.full_like(qt, float("nan"))
            hip.call("ttm_sdpa", hip.ptr(qt), hip.ptr(kt), hip.ptr(vt), None, 1, hip.ptr(out), hip.BF16, B, Hq, Hkv, S, S, D, 1, 0.0,
                     hip.current_stream())
            res[variant] = untilize_dev(hip, out, q.shape, dev).float().cpu().numpy()
    finally:
        hip.set_option("sdpa_variant", 0)
    orc.set_threads(orc.max_threads())
    try:
        want = orc.sdpa(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, is_causal=True)
    finally:
        orc.set_threads(1)
    assert np.array_equal(res[0], res[7])        # 768 blocks on 256 CUs: the automatic choice is the four-wavefront form
    for variant in (7, 8):
        assert np.all(np.isfinite(res[variant]))
        assert np.max(np.abs(res[variant] - want)) <= 2.0 ** -6
        assert metrics.get_pcc(want, res[variant]) >= 0.9999
        assert np.array_equal(res[variant][:, :, 0, :], np.repeat(v.float().numpy()[:, :, 0, :], Hq // Hkv, axis=1))


@pytest.mark.parametrize("variant", [0, 1, 4, 6, 7])
@pytest.mark.parametrize("flags", [15, 1, 6, 8, 9])
@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal", [(1, 8, 2, 256, 256, 128, True), (2, 4, 4, 96, 160, 64, False), (1, 4, 1, 70, 70, 32, True),
                                                      (1, 2, 2, 40, 300, 256, False)])
def test_sdpa_heads_inner_equals_the_head_major_call(hip, dev, B, Hq, Hkv, Sq, Sk, D, causal, flags, variant):
    """ttm_sdpa_heads_inner with q / k / v / out (any subset, by flag) laid out [B, S, H * D], heads side by side, against
    ttm_sdpa on [B, H, S, D]: both layouts hold the same tiles in another order, so the results are identical bit for
    bit once the output is brought back to one shape."""
    q = datagen.randn((B, Hq, Sq, D), seed=22, dtype=torch.bfloat16)
    k = datagen.randn((B, Hkv, Sk, D), seed=23, dtype=torch.bfloat16)
    v = datagen.randn((B, Hkv, Sk, D), seed=24, dtype=torch.bfloat16)
    inner = lambda t: t.permute(0, 2, 1, 3).reshape(t.shape[0], t.shape[2], t.shape[1] * t.shape[3]).contiguous()
    hip.set_option("sdpa_variant", variant)
    try:
        qt, kt, vt = (tilize_dev(hip, t, dev) for t in (q, k, v))
        want_t = torch.full_like(qt, float("nan"))
        hip.call("ttm_sdpa", hip.ptr(qt), hip.ptr(kt), hip.ptr(vt), None, 1, hip.ptr(want_t), hip.BF16, B, Hq, Hkv, Sq, Sk, D, int(causal), 0.0,
                 hip.current_stream())
        want = untilize_dev(hip, want_t, q.shape, dev).cpu()
        qi = tilize_dev(hip, inner(q), dev) if flags & 1 else qt
        ki = tilize_dev(hip, inner(k), dev) if flags & 2 else kt
        vi = tilize_dev(hip, inner(v), dev) if flags & 4 else vt
        out = torch.full_like(qt, float("nan"))
        hip.call("ttm_sdpa_heads_inner", hip.ptr(qi), hip.ptr(ki), hip.ptr(vi), None, 1, hip.ptr(out), hip.BF16, B, Hq, Hkv, Sq, Sk, D, int(causal),
                 0.0, flags, hip.current_stream())
    finally:
        hip.set_option("sdpa_variant", 0)
    if flags & 8:
        got = untilize_dev(hip, out, (B, Sq, Hq * D), dev).cpu().reshape(B, Sq, Hq, D).permute(0, 2, 1, 3)
    else:
        got = untilize_dev(hip, out, q.shape, dev).cpu()
    torch.cuda.synchronize()
    assert torch.equal(got, want)


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 6, 7])
@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal,window,sink,mask,flags", [
    (1, 4, 2, 256, 256, 128, True, 64, False, None, 0), (1, 4, 2, 256, 256, 128, True, 1, False, None, 0),
    (1, 4, 2, 300, 300, 64, True, 100, True, None, 0), (2, 2, 2, 96, 160, 128, False, 40, False, None, 0),
    (1, 2, 1, 200, 200, 32, False, 0, False, None, 0), (1, 2, 2, 160, 160, 64, False, 65, True, "b1", 0),
    (1, 8, 2, 512, 512, 128, True, 129, True, None, 15), (1, 2, 2, 70, 70, 64, True, 1000, True, None, 0),
    (1, 4, 2, 128, 2048, 128, False, 600, True, None, 0), (1, 4, 4, 96, 1536, 64, True, 200, True, None, 9),   # key shares
    (1, 2, 2, 128, 128, 128, True, None, True, None, 0), (2, 3, 3, 64, 100, 64, False, None, True, "bh", 0),
    (1, 1, 1, 100, 300, 256, False, 33, True, None, 0), (1, 4, 4, 640, 640, 64, True, 32, False, None, 9),
    (1, 2, 2, 1024, 1024, 128, True, 200, True, None, 0),
    # one mask shared by a batch of three, per head and for all heads
    (3, 2, 2, 96, 128, 64, False, None, False, "1h", 0), (3, 4, 2, 64, 64, 128, False, 20, True, "11", 0)])
def test_sdpa_sliding_window_and_attention_sink(hip, dev, orc, B, Hq, Hkv, Sq, Sk, D, causal, window, sink, mask, flags, variant):
    """ttm_sdpa_windowed against the oracle: causal windows (one key, shorter and longer than a 64-key pass, longer than
    the sequence), symmetric windows, width 0, with and without the per-head sink, with a mask on top, ragged lengths,
    head-inner layouts, all three kernel variants."""
    if variant == 1 and Sq * Sk >= 512 * 512:
        pytest.skip("the 32-key kernel is covered by the small shapes")
    import oracle.metrics as metrics
    q = datagen.randn((B, Hq, Sq, D), seed=112, dtype=torch.bfloat16)
    k = datagen.randn((B, Hkv, Sk, D), seed=113, dtype=torch.bfloat16)
    v = datagen.randn((B, Hkv, Sk, D), seed=114, dtype=torch.bfloat16)
    m = datagen.randn((1 if mask[0] == "1" else B, 1 if mask[1] == "1" else Hq, Sq, Sk), seed=115, dtype=torch.bfloat16) if mask else None
    sk = (datagen.randn((1, Hq, 1, 1), seed=116, dtype=torch.bfloat16) * 8).contiguous() if sink else None
    inner = lambda t: t.permute(0, 2, 1, 3).reshape(t.shape[0], t.shape[2], t.shape[1] * t.shape[3]).contiguous()
    qt = tilize_dev(hip, inner(q) if flags & 1 else q, dev)
    kt = tilize_dev(hip, inner(k) if flags & 2 else k, dev)
    vt = tilize_dev(hip, inner(v) if flags & 4 else v, dev)
    mt = tilize_dev(hip, m, dev) if m is not None else None
    st = tilize_dev(hip, sk, dev) if sink else None
    out = torch.full_like(qt, float("nan"))
    hip.set_option("sdpa_variant", variant)
    try:
        hip.call("ttm_sdpa_windowed", hip.ptr(qt), hip.ptr(kt), hip.ptr(vt), hip.ptr(mt) if mt is not None else None,
                 m.shape[1] if m is not None else 1, m.shape[0] if m is not None else 1, hip.ptr(out), hip.BF16, B, Hq, Hkv, Sq, Sk, D,
                 int(causal), 0.0, flags, -1 if window is None else window, hip.ptr(st) if sink else None, hip.current_stream())
    finally:
        hip.set_option("sdpa_variant", 0)
    if flags & 8:
        res = untilize_dev(hip, out, (B, Sq, Hq * D), dev).cpu().reshape(B, Sq, Hq, D).permute(0, 2, 1, 3)
    else:
        res = untilize_dev(hip, out, q.shape, dev).cpu()
    torch.cuda.synchronize()
    res = res.float().numpy()
    want = orc.sdpa(q.float().numpy(), k.float().numpy(), v.float().numpy(), None if m is None else m.float().numpy(),
                    is_causal=causal, sliding_window=window, attention_sink=None if sk is None else sk.float().numpy())
    assert np.all(np.isfinite(out.float().cpu().numpy()))
    # probabilities are rounded to bf16 before P.V (relative 2^-9 each) and the output once more
    assert np.max(np.abs(res - want)) <= 2.0 ** -6
    assert metrics.get_pcc(want, res) >= 0.9999
    if window is not None and window < Sk and not sink:
        plain = orc.sdpa(q.float().numpy(), k.float().numpy(), v.float().numpy(), None if m is None else m.float().numpy(), is_causal=causal)
        assert np.max(np.abs(plain - want)) > 0.05          # the window matters for this case


def test_sdpa_window_does_not_read_keys_outside_it(hip, dev, orc):
    """Causal window of 64 keys over 1024: key tiles wholly in front of a query block's window hold NaN in K and Inf in V
    for the queries of the last block; the result for those queries is finite and equal to the oracle's on clean data."""
    B, H, S, D, w = 1, 2, 1024, 128, 64
    q = datagen.randn((B, H, S, D), seed=120, dtype=torch.bfloat16)
    k = datagen.randn((B, H, S, D), seed=121, dtype=torch.bfloat16)
    v = datagen.randn((B, H, S, D), seed=122, dtype=torch.bfloat16)
    kb, vb = k.clone(), v.clone()
    first_q = S - 128                                       # the last block of 128 queries
    hidden = (first_q - w + 1) // 32 * 32                   # keys no query of that block sees
    kb[:, :, :hidden], vb[:, :, :hidden] = float("nan"), float("inf")
    qt, kt, vt = tilize_dev(hip, q, dev), tilize_dev(hip, kb, dev), tilize_dev(hip, vb, dev)
    out = torch.full_like(qt, float("nan"))
    hip.call("ttm_sdpa_windowed", hip.ptr(qt), hip.ptr(kt), hip.ptr(vt), None, 1, 1, hip.ptr(out), hip.BF16, B, H, H, S, S, D, 1, 0.0, 0,
             w, None, hip.current_stream())
    got = untilize_dev(hip, out, q.shape, dev).float().cpu().numpy()[:, :, first_q:]
    want = orc.sdpa(q.float().numpy(), k.float().numpy(), v.float().numpy(), is_causal=True, sliding_window=w)[:, :, first_q:]
    assert np.all(np.isfinite(got)) and np.max(np.abs(got - want)) <= 2.0 ** -6


def _i64(v):
    return np.array(v, dtype=np.int64)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("tiled", [False, True])
@pytest.mark.parametrize("cs,as_,bs", [((3, 40, 70), (3, 40, 70), (3, 40, 70)), ((1, 40, 1), (3, 40, 70), (1, 1, 70)),
                                       ((2, 3, 1, 33), (1, 3, 35, 33), (1,)), ((64, 64), (64, 64), (1, 1)),
                                       ((2, 40, 64), (1, 1, 64), (2, 40, 1)), ((3, 64, 96), (3, 64, 96), (3, 64, 96))])
def test_where_bit_exact(hip, dev, orc, dtype, tiled, cs, as_, bs):
    """ttm_where against the oracle: same-shape and broadcasting operands (condition, either value, a scalar), ragged
    tiles whose padding must stay zero, both layouts and dtypes; NaN and -0.0 in the condition; the values move as bits."""
    rank = max(len(cs), len(as_), len(bs))
    pad = lambda s: (1,) * (rank - len(s)) + tuple(s)
    os_ = tuple(max(x) for x in zip(pad(cs), pad(as_), pad(bs)))
    c = (datagen.randn(pad(cs), seed=150, dtype=dtype) > 0).to(dtype)
    c.view(-1)[0], c.view(-1)[1] = float("nan"), -0.0
    a = datagen.randn(pad(as_), seed=151, dtype=dtype)
    b = datagen.randn(pad(bs), seed=152, dtype=dtype)
    a.view(-1)[0] = float("inf")
    code, lay = (hip.BF16 if dtype == torch.bfloat16 else hip.F32), (hip.TILE if tiled else hip.ROW_MAJOR)
    put = (lambda t: tilize_dev(hip, t, dev)) if tiled else (lambda t: t.contiguous().to(dev))
    ct, at, bt = put(c), put(a), put(b)
    n = int(np.prod(os_[:-2], dtype=np.int64)) * ((os_[-2] + 31) // 32 * 32) * ((os_[-1] + 31) // 32 * 32) if tiled else int(np.prod(os_))
    out = torch.full((n,), float("nan"), dtype=dtype, device=dev)
    shapes = [_i64(pad(cs)), _i64(pad(as_)), _i64(pad(bs)), _i64(os_)]           # kept alive across the call
    hip.call("ttm_where", hip.ptr(ct), shapes[0].ctypes.data, hip.ptr(at), shapes[1].ctypes.data, hip.ptr(bt),
             shapes[2].ctypes.data, hip.ptr(out), shapes[3].ctypes.data, rank, code, lay, hip.current_stream())
    got = untilize_dev(hip, out, os_, dev).cpu() if tiled else out.reshape(os_).cpu()
    torch.cuda.synchronize()
    want = orc.where(c.float().numpy(), a.float().numpy(), b.float().numpy())
    assert np.array_equal(got.float().numpy(), np.broadcast_to(want, os_), equal_nan=True)
    if tiled:
        back = tilize_dev(hip, got, dev)
        assert torch.equal(back.view(torch.int16 if dtype == torch.bfloat16 else torch.int32), out.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,vocab,dim,unsigned", [(64, 1000, 4096, False), (7, 33, 24, True), (300, 50, 5, False), (1, 1, 8, False)])
def test_embedding_bit_exact(hip, dev, orc, dtype, rows, vocab, dim, unsigned):
    """ttm_embedding against the oracle: wide and narrow rows (16-byte and element-wise paths), indices below 0 and past the
    table (clamped, tools/golden/mapping.py:2910-2911), UInt32 indices."""
    g = torch.Generator().manual_seed(160)
    w = datagen.randn((vocab, dim), seed=161, dtype=dtype)
    idx = torch.randint(0, vocab, (rows,), generator=g, dtype=torch.int32)
    if rows > 3:
        idx[1] = vocab + 5
        if not unsigned:
            idx[2] = -3
    wd, idd = w.to(dev), idx.to(dev)
    out = torch.full((rows, dim), float("nan"), dtype=dtype, device=dev)
    hip.call("ttm_embedding", hip.ptr(idd), hip.U32 if unsigned else hip.I32, hip.ptr(wd), hip.ptr(out), w.element_size(), rows, vocab, dim,
             hip.current_stream())
    torch.cuda.synchronize()
    want = orc.embedding(idx.numpy(), w.float().numpy())
    assert np.array_equal(out.float().cpu().numpy(), want)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,cols", [(32, 128256), (5, 63), (1, 1), (9, 64), (130, 1000), (7, 50003), (600, 8192), (3, 8193)])
def test_argmax_first_largest(hip, dev, orc, dtype, rows, cols):
    """ttm_argmax against the oracle: a vocabulary-sized row (the two-step kernel; rows of whole 16-byte groups and not),
    fewer columns than lanes, ties (bf16 rows of 128 256 random values have many; the first index wins, also across the
    slices of a row), NaNs (count as largest, the first one wins), -inf rows."""
    x = datagen.randn((rows, cols), seed=170, dtype=dtype)
    if cols > 40:
        x[0, 7] = x[0, 33] = 50.0
        if rows > 1:
            x[1, 20] = float("nan")
        if rows > 2:
            x[2, :] = float("-inf")
    if cols > 8000:   # the same maximum in the first and in the last slice; NaNs in two slices; a maximum in the last column
        if rows > 3:
            x[3, 100] = x[3, cols - 5] = 60.0
        if rows > 4:
            x[4, cols - 3] = x[4, 4000] = float("nan")
        if rows > 5:
            x[5, cols - 1] = 70.0
    xd = x.to(dev)
    out = torch.full((rows,), -1, dtype=torch.int32, device=dev)
    hip.call("ttm_argmax", hip.ptr(xd), hip.BF16 if dtype == torch.bfloat16 else hip.F32, hip.ptr(out), rows, cols, hip.current_stream())
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), orc.argmax(x.float().numpy(), -1))
    assert np.array_equal(out.cpu().numpy(), torch.argmax(x.float(), dim=-1).numpy())


@pytest.mark.parametrize("start,end,step", [(0, 2048, 1), (3, 40, 4), (5, -5, -2), (0, 1, 0.125), (0, 70000, 7)])
def test_arange_all_dtypes(hip, dev, orc, start, end, step):
    n = int(np.ceil((end - start) / step))
    for code, tdt, ndt in ((hip.F32, torch.float32, np.float32), (hip.BF16, torch.bfloat16, None), (hip.I32, torch.int32, np.int32),
                           (hip.U32, torch.int32, np.uint32)):
        if code == hip.U32 and (start < 0 or end < 0):
            continue
        out = torch.zeros((n,), dtype=tdt, device=dev)
        hip.call("ttm_arange", hip.ptr(out), code, n, float(start), float(step), hip.current_stream())
        torch.cuda.synchronize()
        want = torch.arange(start, end, step, dtype=torch.float32)
        if ndt is None:
            assert torch.equal(out.cpu(), want.to(torch.bfloat16))
        else:
            assert np.array_equal(out.cpu().numpy().view(ndt), orc.arange(start, end, step, ndt))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("name,code", [("maximum", 100), ("minimum", 101), ("remainder", 102), ("pow", 103), ("atan2", 104)])
def test_binary_composites(hip, dev, orc, dtype, name, code):
    """Maximum / Minimum / Remainder / Pow / Atan2 through ttm_eltwise_binary (op = 100 + EltwiseBinaryCompositeOpType),
    broadcasting a row against a matrix in tiles: max / min / remainder exact after the store rounding, pow and atan2 within
    2 ulp of fp32 before it."""
    a = datagen.randn((70, 96), seed=180, dtype=dtype) * 3
    b = datagen.randn((1, 96), seed=181, dtype=dtype) * 2
    if name == "pow":
        a = a.abs() + 0.1
    a[0, 0] = float("nan")
    at, bt = tilize_dev(hip, a, dev), tilize_dev(hip, b, dev)
    out = torch.full_like(at, float("nan"))
    sa, sb = _i64([70, 96]), _i64([1, 96])                                       # kept alive across the call
    hip.call("ttm_eltwise_binary", code, hip.ptr(at), sa.ctypes.data, hip.ptr(bt), sb.ctypes.data, hip.ptr(out),
             sa.ctypes.data, 2, hip.BF16 if dtype == torch.bfloat16 else hip.F32, hip.TILE, hip.current_stream())
    got = untilize_dev(hip, out, (70, 96), dev).cpu()
    torch.cuda.synchronize()
    want = torch.from_numpy(orc.binary_composite(name, a.float().numpy(), b.float().numpy())).to(dtype)
    if name in ("maximum", "minimum", "remainder"):
        assert np.array_equal(got.float().numpy(), want.float().numpy(), equal_nan=True)
    else:
        assert torch.allclose(got.float(), want.float(), rtol=2.0 ** -7 if dtype == torch.bfloat16 else 1e-5, atol=1e-6, equal_nan=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("tiled", [False, True])
def test_clamp_bit_exact(hip, dev, orc, dtype, tiled):
    """ttm_clamp (ClampScalar) against the oracle: NaN kept, infinities clamped, tile padding left at zero even when the
    lower bound is positive."""
    x = datagen.randn((2, 40, 50), seed=190, dtype=dtype) * 4
    x[0, 0, :3] = torch.tensor([float("nan"), float("inf"), float("-inf")], dtype=dtype)
    code = hip.BF16 if dtype == torch.bfloat16 else hip.F32
    for lo, hi in ((-1.0, 2.5), (0.5, 3.0)):
        xd = tilize_dev(hip, x, dev) if tiled else x.to(dev)
        out = torch.full_like(xd, float("nan"))
        hip.call("ttm_clamp", hip.ptr(xd), hip.ptr(out), code, hip.TILE if tiled else hip.ROW_MAJOR, 2, 40, 50, lo, hi, hip.current_stream())
        got = untilize_dev(hip, out, x.shape, dev).cpu() if tiled else out.cpu()
        torch.cuda.synchronize()
        want = orc.clamp(x.float().numpy(), lo, hi)
        assert np.array_equal(got.float().numpy(), want, equal_nan=True)
        if tiled:
            assert torch.equal(tilize_dev(hip, got, dev).view(torch.uint8), out.view(torch.uint8))       # padding is zero
    with pytest.raises(hip.TTMError, match="ttm_clamp"):
        hip.call("ttm_eltwise_unary", 101, hip.ptr(xd), hip.ptr(out), code, hip.ROW_MAJOR, 2, 40, 50, 0.0, hip.current_stream())
