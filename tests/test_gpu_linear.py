"""GPU parity: ttm_linear (bf16 x bf16 / bfp8_b / bfp4_b, fused bias + activation) against the CPU
oracle on identical seeded inputs.  Tolerances (north star): PCC >= 0.99; the max-abs error is
asserted per weight dtype below.  The oracle multiplies the *dequantised* weights, so the
comparison isolates the kernel (accumulation order, bf16 output rounding, fast GELU), not the
block-float quantisation error; that is covered separately against the unquantised weights with
the reference's own bars (PCC 0.99 bfp8 / 0.98 bfp4, test_weight_dtype_conversion.py:39,78)."""
import numpy as np
import pytest
import torch

from ttmlir_amd import datagen

pytestmark = pytest.mark.gpu


def tilize_dev(hip, t, dev):
    """[.., R, C] torch tensor (2 or 4 byte dtype) -> device tensor in tile order."""
    t = t.contiguous().to(dev)
    b = int(np.prod(t.shape[:-2], dtype=np.int64))
    r, c = t.shape[-2], t.shape[-1]
    pr, pc = (r + 31) // 32 * 32, (c + 31) // 32 * 32
    out = torch.zeros(b * pr * pc, dtype=t.dtype, device=dev)
    hip.call("ttm_tilize", hip.ptr(t), hip.ptr(out), b, r, c, t.element_size(), hip.current_stream())
    return out


def untilize_dev(hip, t, shape, dev):
    b = int(np.prod(shape[:-2], dtype=np.int64))
    out = torch.empty(shape, dtype=t.dtype, device=dev)
    hip.call("ttm_untilize", hip.ptr(t), hip.ptr(out), b, shape[-2], shape[-1], t.element_size(), hip.current_stream())
    return out


def pack_weight(hip, w_f32, fmt, dev):
    K, N = w_f32.shape[-2:]
    b = int(np.prod(w_f32.shape[:-2], dtype=np.int64))
    nt = b * ((K + 31) // 32) * ((N + 31) // 32)
    out = torch.empty(nt * hip.bfp_tile_bytes(fmt), dtype=torch.uint8, device=dev)
    wd = w_f32.contiguous().to(dev)
    hip.call("ttm_bfp_pack", hip.ptr(wd), hip.F32, hip.ROW_MAJOR, hip.ptr(out), fmt, b, K, N, hip.current_stream())
    return out


def run_linear(hip, dev, a, w, bias, act, wfmt, transpose_w=False, bias_tiled=True):
    """a [..,M,K] bf16, w [..,K,N] f32 (or [..,N,K] when transpose_w); returns [..,M,N] bf16 on the host
    together with the weights the kernel actually multiplied (dequantised, [..,K,N])."""
    M, K = a.shape[-2:]
    N = w.shape[-2] if transpose_w else w.shape[-1]
    batch = int(np.prod(a.shape[:-2], dtype=np.int64))
    wbatch = int(np.prod(w.shape[:-2], dtype=np.int64))
    at = tilize_dev(hip, a, dev)
    if wfmt == hip.BF16:
        wq = w.to(torch.bfloat16)
        wt = tilize_dev(hip, wq, dev)
        w_eff = wq.float()
    else:
        wt = pack_weight(hip, w, wfmt, dev)
        back = torch.empty(w.shape, dtype=torch.float32, device=dev)
        hip.call("ttm_bfp_unpack", hip.ptr(wt), wfmt, hip.ptr(back), hip.F32, hip.ROW_MAJOR, wbatch, K, N,
                 hip.current_stream())
        w_eff = back.cpu()
    bt = None
    if bias is not None:
        bt = tilize_dev(hip, bias.reshape(1, -1), dev) if bias_tiled else bias.to(dev)
    Mp, Np = (M + 31) // 32 * 32, (N + 31) // 32 * 32
    out = torch.full((batch * Mp * Np,), float("nan"), dtype=torch.bfloat16, device=dev)
    hip.call("ttm_linear", hip.ptr(at), hip.BF16, hip.ptr(wt), wfmt, int(transpose_w),
             hip.ptr(bt) if bt is not None else None, hip.BF16, hip.TILE if bias_tiled else hip.ROW_MAJOR,
             hip.ptr(out), hip.BF16, batch, wbatch, M, N, K, hip.ACT[act], hip.current_stream())
    res = untilize_dev(hip, out, tuple(a.shape[:-2]) + (M, N), dev)
    torch.cuda.synchronize()
    return res.cpu(), (w_eff.transpose(-1, -2) if transpose_w else w_eff)


def check(orc, metrics, got_bf16, a, w_eff, bias, act, max_abs, pcc=0.99):
    a32 = a.float().numpy()
    if a32.ndim == 2:
        want = orc.linear(a32, w_eff.numpy(), None if bias is None else bias.float().numpy(), act)
    else:
        want = orc.matmul(a32, w_eff.numpy())
        assert bias is None and act is None
    want = orc.round_bf16(want)                      # the CPU path casts f32 back to bf16 at the end
    got = got_bf16.float().numpy()
    assert np.all(np.isfinite(got))
    err = float(np.max(np.abs(got - want)))
    p = metrics.get_pcc(want, got)
    assert p >= pcc, "pcc %.5f" % p
    assert err <= max_abs, "max abs err %.4g > %.4g" % (err, max_abs)
    return err, p


@pytest.fixture(scope="module")
def metrics():
    import oracle.metrics as m
    return m


def test_c1_bf16_matmul(hip, dev, orc, metrics):
    a, b = datagen.c1_matmul()
    got, w_eff = run_linear(hip, dev, a, b.float(), None, None, hip.BF16)
    # |C| ~ sqrt(512) ~ 23 -> bf16 half-ulp 0.0625 at 16..32; allow one bf16 ulp (0.25 at 32..64)
    check(orc, metrics, got, a, w_eff, None, None, max_abs=0.25)


@pytest.mark.parametrize("wfmt_name", ["bfp8", "bfp4", "bf16"])
@pytest.mark.parametrize("M,K,N,act,bias", [
    (256, 512, 256, None, False), (256, 256, 512, "gelu", True), (512, 128, 256, "silu", True),
    (64, 96, 160, "sigmoid", True), (32, 512, 64, "gelu", True), (17, 200, 100, "relu", True),
    (288, 64, 320, "gelu", True), (1, 64, 32, None, True)])
def test_linear_shapes(hip, dev, orc, metrics, wfmt_name, M, K, N, act, bias):
    wfmt = {"bfp8": hip.BFP8B, "bfp4": hip.BFP4B, "bf16": hip.BF16}[wfmt_name]
    a = datagen.randn((M, K), seed=M + K, dtype=torch.bfloat16)
    w = datagen.randn((K, N), seed=N, std=0.05)
    b = datagen.randn((N,), seed=7, std=0.5, dtype=torch.bfloat16) if bias else None
    got, w_eff = run_linear(hip, dev, a, w, b, act, wfmt)
    # outputs are O(1); one bf16 ulp at |y| < 4 is 2^-6... allow 2^-5 for accumulation-order effects
    check(orc, metrics, got, a, w_eff, b, act, max_abs=2.0 ** -5)


def test_linear_row_major_bias_and_transposed_weights(hip, dev, orc, metrics):
    a = datagen.randn((96, 128), seed=1, dtype=torch.bfloat16)
    w = datagen.randn((128, 192), seed=2, std=0.05)
    b = datagen.randn((192,), seed=3, std=0.5, dtype=torch.bfloat16)
    got, w_eff = run_linear(hip, dev, a, w, b, "gelu", hip.BFP8B, bias_tiled=False)
    check(orc, metrics, got, a, w_eff, b, "gelu", max_abs=2.0 ** -5)
    for M in (96, 32):
        a = datagen.randn((M, 128), seed=1, dtype=torch.bfloat16)
        got, w_eff = run_linear(hip, dev, a, w.t().contiguous(), b, None, hip.BF16, transpose_w=True)
        check(orc, metrics, got, a, w_eff, b, None, max_abs=2.0 ** -5)


def test_batched_matmul(hip, dev, orc, metrics):
    a = datagen.randn((2, 3, 64, 96), seed=4, dtype=torch.bfloat16)
    w = datagen.randn((2, 3, 96, 64), seed=5, std=0.1)
    got, w_eff = run_linear(hip, dev, a, w, None, None, hip.BF16)
    check(orc, metrics, got, a, w_eff, None, None, max_abs=2.0 ** -5)
    w1 = datagen.randn((1, 96, 64), seed=6, std=0.1)          # RHS with a single batch broadcasts
    got, w_eff = run_linear(hip, dev, a, w1, None, None, hip.BF16)
    want = orc.round_bf16(orc.matmul(a.float().numpy(), w_eff.numpy()))
    assert np.max(np.abs(got.float().numpy() - want)) <= 2.0 ** -5


@pytest.mark.parametrize("M", [32, 2048])
def test_c3_linear_full_size(hip, dev, orc, metrics, M):
    """Config 3 at full size, every one of the M x 14336 outputs against the oracle (all host cores: 240 GFLOP at
    M = 2048)."""
    a, w, bias = datagen.c3_linear(M)
    got, w_eff = run_linear(hip, dev, a, w, bias, "gelu", hip.BFP8B)
    orc.set_threads(orc.max_threads())
    try:
        want = orc.round_bf16(orc.linear(a.float().numpy(), w_eff.contiguous().numpy(), bias.float().numpy(), "gelu"))
    finally:
        orc.set_threads(1)
    g = got.float().numpy()
    assert g.shape == want.shape == (M, 14336)
    # |y| up to ~6 -> bf16 ulp 2^-5; accumulation over K=4096 in a different order adds less than that
    assert np.max(np.abs(g - want)) <= 2.0 ** -5
    assert metrics.get_pcc(want, g) >= 0.9999
    assert np.mean(g == want) >= 0.98                  # the rest are single bf16 roundings at ties
    # quantisation itself against the unquantised weights: the reference's own bar for bfp8 weights
    rows = slice(0, 32) if M == 32 else slice(1000, 1032)
    ref = torch.nn.functional.gelu(a[rows].float() @ w + bias.float())
    assert metrics.get_pcc(ref.numpy(), g[rows]) >= 0.99
    # linearity in the activations at full size: f(2a) - 2 f(a) == 0 without bias/activation (exact in bf16/f32)
    g1, _ = run_linear(hip, dev, a, w, None, None, hip.BFP8B)
    g2, _ = run_linear(hip, dev, (a.float() * 2).to(torch.bfloat16), w, None, None, hip.BFP8B)
    assert torch.equal(g2.float(), g1.float() * 2)


@pytest.mark.parametrize("wfmt_name,bar", [("bfp8", 0.99), ("bfp4", 0.98)])
def test_weight_dtype_bars(hip, dev, metrics, wfmt_name, bar):
    """test/python/golden/ttir_ops/matmul/test_weight_dtype_conversion.py:15-88 shapes, PCC vs torch."""
    wfmt = {"bfp8": hip.BFP8B, "bfp4": hip.BFP4B}[wfmt_name]
    a = datagen.randn((64, 128), seed=0, dtype=torch.bfloat16)
    w = datagen.randn((128, 64), seed=1)
    got, _ = run_linear(hip, dev, a, w, None, None, wfmt)
    ref = a.float() @ w.to(torch.bfloat16).float()
    assert metrics.get_pcc(ref.numpy(), got.float().numpy()) >= bar


@pytest.mark.parametrize("wfmt_name", ["bfp8", "bfp4"])
@pytest.mark.parametrize("option,value", [("linear_ntw", 4), ("linear_ntw", 3), ("linear_ntw", 2), ("linear_split_k", 2),
                                          ("linear_split_k", 3), ("linear_variant", 1), ("linear_variant", 5)])
def test_block_float_kernel_configurations(hip, dev, orc, metrics, wfmt_name, option, value):
    """Every block width of the LDS-direct kernel, the split-K path with its reduction kernel, the register-staged
    kernel and the 64-bit-addressed fallback, on a ragged shape with an odd number of k-tiles."""
    wfmt = {"bfp8": hip.BFP8B, "bfp4": hip.BFP4B}[wfmt_name]
    M, K, N = 330, 7 * 32 + 8, 21 * 32 + 5
    a = datagen.randn((M, K), seed=11, dtype=torch.bfloat16)
    w = datagen.randn((K, N), seed=12, std=0.05)
    b = datagen.randn((N,), seed=13, std=0.5, dtype=torch.bfloat16)
    hip.set_option(option, value)
    try:
        got, w_eff = run_linear(hip, dev, a, w, b, "gelu", wfmt)
    finally:
        hip.set_option(option, 0)
    check(orc, metrics, got, a, w_eff, b, "gelu", max_abs=2.0 ** -5)


@pytest.mark.parametrize("wfmt_name", ["bfp8", "bfp4"])
@pytest.mark.parametrize("split", [0, 1, 3, 5])
def test_decode_kernel_k_slices(hip, dev, orc, metrics, wfmt_name, split):
    """M <= 32 path: split-K of the weight-streaming kernel (fp32 partials + reduction with bias and activation), forced
    to several slice counts and left automatic, on a ragged K with a tail tile and a batch of two."""
    wfmt = {"bfp8": hip.BFP8B, "bfp4": hip.BFP4B}[wfmt_name]
    M, K, N = 19, 37 * 32 + 11, 5 * 32 + 7
    a = datagen.randn((2, M, K), seed=41, dtype=torch.bfloat16)
    w = datagen.randn((2, K, N), seed=42, std=0.05)
    b = datagen.randn((N,), seed=43, std=0.5, dtype=torch.bfloat16)
    hip.set_option("linear_decode_split", split)
    try:
        got, w_eff = run_linear(hip, dev, a, w, b, "silu", wfmt)
    finally:
        hip.set_option("linear_decode_split", 0)
    for i in range(2):   # the oracle's linear takes one matrix at a time
        check(orc, metrics, got[i], a[i], w_eff[i], b, "silu", max_abs=2.0 ** -5)


@pytest.mark.parametrize("wfmt_name", ["bfp8", "bfp4"])
@pytest.mark.parametrize("M,K,N", [(32, 1024, 512), (7, 37 * 32 + 11, 5 * 32 + 7)])
def test_decode_kernel_operand_constructions_agree(hip, dev, orc, metrics, wfmt_name, M, K, N):
    """The decode kernel builds its bf16 weight operands either by int -> float conversion (linear_decode_variant 1) or
    as two bit-built terms whose difference is the weight (default).  Weights with whole zero rows (exponent 0), rows of
    x100 outliers (small magnitudes beside a large exponent) and both signs: each route against the oracle, and the two
    against each other within one bf16 step of the result."""
    wfmt = {"bfp8": hip.BFP8B, "bfp4": hip.BFP4B}[wfmt_name]
    a = datagen.randn((M, K), seed=46, dtype=torch.bfloat16)
    w = datagen.randn((K, N), seed=47, std=0.05)
    w[5:9] = 0.0
    w[40:44, ::3] *= 100.0
    w[:, 17] = 0.0
    b = datagen.randn((N,), seed=48, std=0.5, dtype=torch.bfloat16)
    res = {}
    for variant in (1, 0):
        hip.set_option("linear_decode_variant", variant)
        try:
            res[variant], w_eff = run_linear(hip, dev, a, w, b, None, wfmt)
        finally:
            hip.set_option("linear_decode_variant", 0)
        check(orc, metrics, res[variant], a, w_eff, b, None, max_abs=2.0 ** -4)
    x, y = res[0].float(), res[1].float()
    # one bf16 step of the result, plus the fp32 accumulation error, which scales with the summands and not with the
    # (possibly cancelling) sum: 2^-16 of sum |a| |w| is a loose bound for either route
    summands = a.float().abs() @ w_eff.abs()
    step = torch.maximum(x.abs(), y.abs()) * 2.0 ** -7 + summands * 2.0 ** -16 + 1e-6
    assert torch.all((x - y).abs() <= step)
    assert (x != y).float().mean().item() < 0.01


def test_decode_kernel_splits_narrow_outputs_by_itself(hip, dev, orc, metrics):
    """[32, 4096] x bfp4_b [4096, 1024]: 16 column groups on a 256-CU device -> the launcher slices K."""
    a = datagen.randn((32, 4096), seed=44, dtype=torch.bfloat16)
    w = datagen.randn((4096, 1024), seed=45, std=0.02)
    got, w_eff = run_linear(hip, dev, a, w, None, None, hip.BFP4B)
    check(orc, metrics, got, a, w_eff, None, None, max_abs=2.0 ** -5)


@pytest.mark.parametrize("wfmt_name", ["bfp8", "bfp4"])
def test_two_part_grid_with_ragged_remainder(hip, dev, orc, metrics, wfmt_name):
    """The optional two-part grid: 300 column blocks and a bit on a 256-CU device run as one full round of 8-tile-wide
    blocks plus the remaining 353 column tiles (the last one ragged) in 6-tile-wide blocks of the same launch.  Compared with the single-part grid bit for bit
    (same per-element accumulation order) and with the oracle on three column bands."""
    wfmt = {"bfp8": hip.BFP8B, "bfp4": hip.BFP4B}[wfmt_name]
    M, K, N = 200, 96, 300 * 256 + 40
    a = datagen.randn((M, K), seed=51, dtype=torch.bfloat16)
    w = datagen.randn((K, N), seed=52, std=0.1)
    b = datagen.randn((N,), seed=53, std=0.5, dtype=torch.bfloat16)
    one, w_eff = run_linear(hip, dev, a, w, b, "relu", wfmt)
    hip.set_option("linear_two_part", 1)
    try:
        got, _ = run_linear(hip, dev, a, w, b, "relu", wfmt)
    finally:
        hip.set_option("linear_two_part", 0)
    assert torch.equal(got, one)
    for cols in (slice(0, 512), slice(65536 - 256, 65536 + 256), slice(N - 300, N)):
        check(orc, metrics, got[:, cols], a, w_eff[:, cols].contiguous(), b[cols], "relu", max_abs=2.0 ** -5)

@pytest.mark.parametrize("wfmt_name,M,K,N,option,value", [
    ("bfp8", 32, 1200, 200, None, 0),                   # decode kernel
    ("bfp4", 20, 1200, 200, "linear_decode_split", 3),  # decode kernel with k-slices: activation applied by the reduction
    ("bf16", 32, 256, 96, None, 0),                     # small-M kernel for bf16 weights
    ("bfp8", 330, 232, 677, None, 0),                   # LDS-direct main kernel, ragged
    ("bfp4", 330, 232, 677, "linear_split_k", 2),       # split-K main kernel
    ("bfp8", 512, 256, 2048, "linear_two_pass", 2),     # image pass + matrix pass
    ("bf16", 300, 256, 512, None, 0),                   # bf16 weights through the image route
])
def test_relu_epilogue_keeps_nan(hip, dev, orc, wfmt_name, M, K, N, option, value):
    """linear(..., "relu") on activations that hold a NaN: the rows it reaches stay NaN after the fused relu, as with
    arith.maximumf of the CPU lowering (lib/Conversion/TTIRToLinalg/EltwiseUnary.cpp:508-541) and the oracle; every other
    output is what it is without the NaN, and negative sums become +0.0."""
    wfmt = {"bfp8": hip.BFP8B, "bfp4": hip.BFP4B, "bf16": hip.BF16}[wfmt_name]
    a = datagen.randn((M, K), seed=61, dtype=torch.bfloat16)
    w = datagen.randn((K, N), seed=62, std=0.1)
    b = datagen.randn((N,), seed=63, std=0.5, dtype=torch.bfloat16)
    a[3, 5] = float("nan")
    a[M - 1, K - 1] = float("nan")
    if option:
        hip.set_option(option, value)
    try:
        got, w_eff = run_linear(hip, dev, a, w, b, "relu", wfmt)
    finally:
        if option:
            hip.set_option(option, 0)
    with np.errstate(invalid="ignore"):
        want = orc.round_bf16(orc.linear(a.float().numpy(), w_eff.numpy(), b.float().numpy(), "relu"))
    got = got.float().numpy()
    assert np.isnan(want[3]).all() and np.isnan(want[M - 1]).all() and np.isnan(want).sum() == 2 * N
    assert np.array_equal(np.isnan(got), np.isnan(want)), "NaN rows differ from the oracle's"
    fin = ~np.isnan(want)
    assert np.max(np.abs(got[fin] - want[fin])) <= 2.0 ** -5
    assert not np.signbit(got[fin]).any()                # relu never leaves a -0.0


@pytest.mark.parametrize("tail", ["add", "multiply"])
@pytest.mark.parametrize("wfmt_name,M,K,N,option,value", [
    ("bfp8", 32, 1200, 200, None, 0),                 # decode kernel
    ("bfp4", 20, 1200, 200, "linear_decode_split", 3),  # decode kernel with k-slices: tail applied by the reduction
    ("bf16", 32, 256, 96, None, 0),                   # small-M kernel for bf16 weights
    ("bfp8", 330, 232, 677, None, 0),                 # LDS-direct main kernel, ragged
    ("bfp4", 330, 232, 677, "linear_split_k", 2),     # split-K main kernel
    ("bf16", 288, 160, 320, None, 0),                 # register-staged kernel
    ("bfp8", 96, 96, 160, "linear_variant", 1),       # 64-bit-addressed fallback
])
def test_linear_with_fused_tail_equals_two_ops(hip, dev, orc, metrics, tail, wfmt_name, M, K, N, option, value):
    """ttm_linear_tail (add / multiply with a second tensor in the epilogue) against ttm_linear followed by the oracle's
    binary op on the rounded result: bit exact on every kernel path, because both roundings are kept."""
    wfmt = {"bfp8": hip.BFP8B, "bfp4": hip.BFP4B, "bf16": hip.BF16}[wfmt_name]
    a = datagen.randn((M, K), seed=61, dtype=torch.bfloat16)
    w = datagen.randn((K, N), seed=62, std=0.05)
    b = datagen.randn((N,), seed=63, std=0.5, dtype=torch.bfloat16)
    t = datagen.randn((M, N), seed=64, dtype=torch.bfloat16)
    if option:
        hip.set_option(option, value)
    try:
        plain, _ = run_linear(hip, dev, a, w, b, "silu", wfmt)
        at = tilize_dev(hip, a, dev)
        wt = tilize_dev(hip, w.to(torch.bfloat16), dev) if wfmt == hip.BF16 else pack_weight(hip, w, wfmt, dev)
        bt, tt = tilize_dev(hip, b.reshape(1, -1), dev), tilize_dev(hip, t, dev)
        out = torch.full_like(tt, float("nan"))
        hip.call("ttm_linear_tail", hip.ptr(at), hip.BF16, hip.ptr(wt), wfmt, 0, hip.ptr(bt), hip.BF16, hip.TILE, hip.ptr(out), hip.BF16,
                 1, 1, M, N, K, hip.ACT["silu"], 1 if tail == "add" else 2, hip.ptr(tt), hip.current_stream())
        got = untilize_dev(hip, out, (M, N), dev).cpu()
        torch.cuda.synchronize()
    finally:
        if option:
            hip.set_option(option, 0)
    want = orc.round_bf16(orc.binary(tail, plain.float().numpy(), t.float().numpy()))
    assert np.array_equal(got.float().numpy(), want)
    with pytest.raises(hip.TTMError, match="tail op needs its operand"):
        hip.call("ttm_linear_tail", hip.ptr(at), hip.BF16, hip.ptr(wt), wfmt, 0, None, hip.BF16, hip.TILE, hip.ptr(out), hip.BF16,
                 1, 1, M, N, K, 0, 1, None, hip.current_stream())


def test_split_k_is_chosen_for_long_skinny_reductions(hip, dev, orc, metrics):
    """M = 128, N = 256, K = 8192: one round of blocks would use 2 CUs; the launcher splits K."""
    M, K, N = 128, 8192, 256
    a = datagen.randn((M, K), seed=21, dtype=torch.bfloat16)
    w = datagen.randn((K, N), seed=22, std=0.02)
    got, w_eff = run_linear(hip, dev, a, w, None, None, hip.BFP8B)
    # |y| ~ 0.02 * sqrt(8192) ~ 1.8: one bf16 ulp below 4 is 2^-6; allow 2^-5
    check(orc, metrics, got, a, w_eff, None, None, max_abs=2.0 ** -5)


@pytest.mark.parametrize("split", [0, 2])
def test_batched_block_float_matmul(hip, dev, orc, metrics, split):
    """Batched contraction with per-batch bfp8_b weights and with one shared weight matrix, with and without
    a split reduction (the fp32 partials are laid out per batch entry and k-slice)."""
    a = datagen.randn((3, 96, 160), seed=31, dtype=torch.bfloat16)
    w = datagen.randn((3, 160, 96), seed=32, std=0.1)
    hip.set_option("linear_split_k", split)
    try:
        got, w_eff = run_linear(hip, dev, a, w, None, None, hip.BFP8B)
        check(orc, metrics, got, a, w_eff, None, None, max_abs=2.0 ** -5)
        w1 = datagen.randn((1, 160, 96), seed=33, std=0.1)
        got, w_eff = run_linear(hip, dev, a, w1, None, None, hip.BFP8B)
    finally:
        hip.set_option("linear_split_k", 0)
    want = orc.round_bf16(orc.matmul(a.float().numpy(), w_eff.numpy()))
    assert np.max(np.abs(got.float().numpy() - want)) <= 2.0 ** -5


@pytest.mark.parametrize("wfmt_name", ["bfp8", "bfp4"])
@pytest.mark.parametrize("M,K,N,second_first", [(32, 4096, 1024, False), (20, 1200, 200, True), (330, 232, 677, False),
                                                (2048, 512, 1024, True)])
def test_linear_pair_equals_two_launches(hip, dev, wfmt_name, M, K, N, second_first):
    """ttm_linear_pair (two weight matrices of one shape against the same activations in one launch) against two ttm_linear
    calls: bit exact, whichever of the two allocations lies first in memory (the stride between them is signed)."""
    wfmt = {"bfp8": hip.BFP8B, "bfp4": hip.BFP4B}[wfmt_name]
    a = datagen.randn((M, K), seed=71, dtype=torch.bfloat16)
    ws = [datagen.randn((K, N), seed=72 + i, std=0.05) for i in range(2)]
    want = [run_linear(hip, dev, a, w, None, None, wfmt)[0] for w in ws]
    at = tilize_dev(hip, a, dev)
    wt = [pack_weight(hip, w, wfmt, dev) for w in ws]
    Mp, Np = (M + 31) // 32 * 32, (N + 31) // 32 * 32
    both = torch.full((2, Mp * Np), float("nan"), dtype=torch.bfloat16, device=dev)
    o = [both[1], both[0]] if second_first else [both[0], both[1]]
    hip.call("ttm_linear_pair", hip.ptr(at), hip.ptr(wt[0]), hip.ptr(wt[1]), wfmt, hip.ptr(o[0]), hip.ptr(o[1]), M, N, K,
             hip.current_stream())
    for i in range(2):
        got = untilize_dev(hip, o[i], (M, N), dev).cpu()
        assert torch.equal(got, want[i])
    with pytest.raises(hip.TTMError, match="two distinct"):
        hip.call("ttm_linear_pair", hip.ptr(at), hip.ptr(wt[0]), hip.ptr(wt[0]), wfmt, hip.ptr(o[0]), hip.ptr(o[1]), M, N, K,
                 hip.current_stream())


@pytest.mark.parametrize("wfmt_name", ["bfp8", "bfp4"])
@pytest.mark.parametrize("M,K,N,option,value,act,bias", [
    (330, 200, 677, None, 0, "gelu", True),          # odd number of k-tiles, ragged everywhere
    (330, 232, 677, "linear_split_k", 2, None, False),  # k-slices read the zero image past their end
    (300, 520, 200, "linear_split_k", 4, "silu", True),
    (512, 256, 1024, "linear_ntw", 3, None, True),   # 6-tile-wide blocks: the last block has columns to spare
    (512, 256, 320, "linear_ntw", 2, "relu", False),
    (2048, 512, 2048, None, 0, None, True),
    (512, 256, 1024, "linear_ntw", 7, "gelu", True),  # 7-tile-wide blocks (wide and narrow wavefronts), 32 tiles = 4 x 7 + 4
    (330, 200, 677, "linear_ntw", 7, None, False),   # ragged rows and columns, 22 tiles = 3 x 7 + 1
    (256, 64, 224, "linear_ntw", 7, "silu", True),   # exactly one block
    (2048, 256, 10240, None, 0, "gelu", True),       # more blocks than CUs: several rounds, XCD-aware block order
    (2048, 192, 10240, "linear_ntw", 7, None, True),
    (2080, 256, 9000, "linear_ntw", 4, "relu", False),
])
def test_two_pass_launch_equals_the_fused_kernel(hip, dev, wfmt_name, M, K, N, option, value, act, bias):
    """linear_two_pass = 2 dequantises the weights once into bf16 fragment images and runs the main loop without the
    conversion; = 1 keeps the fused kernel.  Same arithmetic in the same order: bit-identical results."""
    wfmt = {"bfp8": hip.BFP8B, "bfp4": hip.BFP4B}[wfmt_name]
    a = datagen.randn((M, K), seed=81, dtype=torch.bfloat16)
    w = datagen.randn((K, N), seed=82, std=0.05)
    b = datagen.randn((N,), seed=83, std=0.5, dtype=torch.bfloat16) if bias else None
    got = {}
    if option:
        hip.set_option(option, value)
    try:
        for mode in (1, 2):
            hip.set_option("linear_two_pass", mode)
            got[mode], _ = run_linear(hip, dev, a, w, b, act, wfmt)
    finally:
        hip.set_option("linear_two_pass", 0)
        if option:
            hip.set_option(option, 0)
    assert torch.equal(got[1], got[2])


def test_two_pass_launch_with_batches_pairs_and_tails(hip, dev, orc, metrics):
    """The image pass covers every weight set of a launch: per-batch weights, one shared set, a pair of separately
    allocated matrices, and the element-wise tail still runs in the second pass's epilogue."""
    try:
        res = {}
        for mode in (1, 2):
            hip.set_option("linear_two_pass", mode)
            a = datagen.randn((3, 288, 160), seed=91, dtype=torch.bfloat16)
            own, _ = run_linear(hip, dev, a, datagen.randn((3, 160, 96), seed=92, std=0.1), None, None, hip.BFP8B)
            shared, _ = run_linear(hip, dev, a, datagen.randn((1, 160, 96), seed=93, std=0.1), None, None, hip.BFP4B)
            M, K, N = 330, 232, 677
            x = datagen.randn((M, K), seed=94, dtype=torch.bfloat16)
            ws = [pack_weight(hip, datagen.randn((K, N), seed=95 + i, std=0.05), hip.BFP8B, dev) for i in range(2)]
            xt, tt = tilize_dev(hip, x, dev), tilize_dev(hip, datagen.randn((M, N), seed=97, dtype=torch.bfloat16), dev)
            Mp, Np = (M + 31) // 32 * 32, (N + 31) // 32 * 32
            both = torch.full((2, Mp * Np), float("nan"), dtype=torch.bfloat16, device=dev)
            hip.call("ttm_linear_pair", hip.ptr(xt), hip.ptr(ws[1]), hip.ptr(ws[0]), hip.BFP8B, hip.ptr(both[0]), hip.ptr(both[1]), M, N, K,
                     hip.current_stream())
            tail = torch.full((Mp * Np,), float("nan"), dtype=torch.bfloat16, device=dev)
            hip.call("ttm_linear_tail", hip.ptr(xt), hip.BF16, hip.ptr(ws[0]), hip.BFP8B, 0, None, hip.BF16, hip.TILE, hip.ptr(tail), hip.BF16,
                     1, 1, M, N, K, hip.ACT["silu"], 2, hip.ptr(tt), hip.current_stream())
            torch.cuda.synchronize()
            res[mode] = [own, shared, both.cpu(), tail.cpu()]
    finally:
        hip.set_option("linear_two_pass", 0)
    for x, y in zip(res[1], res[2]):
        assert torch.equal(x.view(torch.int16), y.view(torch.int16))   # bit patterns: the padding may hold NaN


@pytest.mark.parametrize("wfmt_name", ["bfp8", "bfp4"])
@pytest.mark.parametrize("M,K,Ns,options", [
    (32, 1024, (512, 128, 128), {"linear_decode_split": 2}),       # decode kernel, k-slices, reduction that knows the members
    (20, 520, (200, 72, 72, 40), {"linear_decode_split": 1}),      # ragged everywhere, four members, direct epilogue
    (64, 256, (96, 160), {"linear_decode_split": 3}),              # two row tiles
    (32, 1024, (512, 128, 128), {"linear_decode_split": 2, "linear_decode_wide": 2}),   # the same with 128 columns per workgroup
    (20, 520, (200, 72, 72, 40), {"linear_decode_split": 1, "linear_decode_wide": 2}),
    (64, 256, (96, 160), {"linear_decode_split": 3, "linear_decode_wide": 2}),
    (330, 232, (677, 100, 300), {"linear_split_k": 1, "linear_two_pass": 1}),   # fused main kernel
    (512, 256, (1024, 256, 256), {"linear_split_k": 1, "linear_two_pass": 2}),  # two passes: one image launch for all members
    (2048, 128, (2048, 512, 512), {"linear_split_k": 1, "linear_two_pass": 2, "linear_ntw": 7}),   # 7-wide blocks, several rounds
    (288, 160, (320, 64), {"linear_split_k": 1, "linear_two_pass": 1, "linear_ntw": 3}),
])
def test_linear_group_equals_separate_launches(hip, dev, wfmt_name, M, K, Ns, options):
    """ttm_linear_group (several weight matrices of different widths against the same activations in one launch) against one
    ttm_linear call per member under the same launch plan: bit exact."""
    import ctypes
    wfmt = {"bfp8": hip.BFP8B, "bfp4": hip.BFP4B}[wfmt_name]
    a = datagen.randn((M, K), seed=101, dtype=torch.bfloat16)
    ws = [datagen.randn((K, N), seed=102 + i, std=0.05) for i, N in enumerate(Ns)]
    for k, v in options.items():
        hip.set_option(k, v)
    try:
        act_names = [(None, "silu", "gelu", "relu")[(i + M) % 4] for i in range(len(Ns))]     # a different activation per member
        want = [run_linear(hip, dev, a, w, None, act, wfmt)[0] for w, act in zip(ws, act_names)]
        at = tilize_dev(hip, a, dev)
        wt = [pack_weight(hip, w, wfmt, dev) for w in ws]
        Mp = (M + 31) // 32 * 32
        outs = [torch.full((Mp * ((N + 31) // 32 * 32),), float("nan"), dtype=torch.bfloat16, device=dev) for N in Ns]
        n = len(Ns)
        wp = (ctypes.c_void_p * n)(*[t.data_ptr() for t in wt])
        op = (ctypes.c_void_p * n)(*[t.data_ptr() for t in outs])
        nn = (ctypes.c_int64 * n)(*Ns)
        acts = (ctypes.c_int * n)(*[hip.ACT[x] for x in act_names])
        hip.call("ttm_linear_group", hip.ptr(at), n, wp, wfmt, op, nn, acts, M, K, hip.current_stream())
        got = [untilize_dev(hip, o, (M, N), dev).cpu() for o, N in zip(outs, Ns)]
        torch.cuda.synchronize()
    finally:
        for k in options:
            hip.set_option(k, 0)
    for g, w in zip(got, want):
        assert torch.equal(g, w)


@pytest.mark.parametrize("wfmt_name", ["bfp8", "bfp4"])
@pytest.mark.parametrize("M,K,N,with_bias,act", [
    (32, 512, 1000, True, "gelu"),       # ragged columns, an even number of column tiles
    (7, 1024, 96, False, "silu"),        # three column tiles: the last workgroup's second tile pair is half there
    (32, 256, 32, True, None),           # one column tile
    (64, 2048, 8256, False, "relu"),     # two row tiles, 129 wide workgroups
    (32, 4096, 28672, True, "gelu"),     # a width at which the wide form is the default
])
def test_decode_kernel_wide_workgroups_equal_narrow_ones(hip, dev, wfmt_name, M, K, N, with_bias, act):
    """The decode kernel with 128 columns per workgroup (linear_decode_wide = 2) against 64 (= 1), neither splitting K: the
    same k order per output, bit-identical results; the default picks one of the two."""
    wfmt = {"bfp8": hip.BFP8B, "bfp4": hip.BFP4B}[wfmt_name]
    a = datagen.randn((M, K), seed=131, dtype=torch.bfloat16)
    w = datagen.randn((K, N), seed=132, std=0.05)
    bias = datagen.randn((1, N), seed=133, dtype=torch.bfloat16) if with_bias else None
    outs = {}
    try:
        hip.set_option("linear_decode_split", 1)
        for wide in (1, 2, 0):
            hip.set_option("linear_decode_wide", wide)
            outs[wide] = run_linear(hip, dev, a, w, bias, act, wfmt)[0]
    finally:
        hip.set_option("linear_decode_split", 0)
        hip.set_option("linear_decode_wide", 0)
    assert torch.equal(outs[1], outs[2]) and torch.equal(outs[0], outs[1])
    assert bool(torch.isfinite(outs[2].float()).all())
