"""Pins the oracle's f32 compute functions against library routines (torch on the CPU) and
closed forms.  Tolerances are those of f32 evaluation order, written per check."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F


def rnd(shape, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(shape) * scale).astype(np.float32)


def test_linear_matches_torch(orc):
    a, b, bias = rnd((37, 53), 0), rnd((53, 29), 1), rnd((29,), 2)
    want = torch.from_numpy(a).double() @ torch.from_numpy(b).double() + torch.from_numpy(bias).double()
    got = orc.linear(a, b, bias)
    assert np.allclose(got, want.numpy(), rtol=1e-5, atol=1e-5)
    # transposes address the stored operand with its last two dims swapped
    assert np.array_equal(orc.linear(a.T.copy(), b, bias, transpose_a=True), got)
    assert np.array_equal(orc.linear(a, b.T.copy(), bias, transpose_b=True), got)
    # the row-streaming variant keeps the same per-element accumulation order: bit identical
    assert np.array_equal(orc.linear(a, b, bias, rowstream=True), got)
    # a dropped bias or a swapped activation order would show here
    g = orc.linear(a, b, bias, act="gelu")
    assert np.allclose(g, F.gelu(want).float().numpy(), rtol=1e-5, atol=1e-5)
    s = orc.linear(a, b, bias, act="silu")
    assert np.allclose(s, F.silu(want).float().numpy(), rtol=1e-5, atol=1e-5)


def test_identity_and_known_matmul(orc):
    a = rnd((8, 8), 3)
    assert np.array_equal(orc.linear(a, np.eye(8, dtype=np.float32)), a)
    x = np.array([[1, 2], [3, 4]], dtype=np.float32)
    y = np.array([[5, 6], [7, 8]], dtype=np.float32)
    assert orc.linear(x, y).tolist() == [[19, 22], [43, 50]]


def test_batched_matmul_broadcast(orc):
    a, b = rnd((2, 3, 5, 7), 4), rnd((1, 7, 4), 5)
    want = torch.from_numpy(a) @ torch.from_numpy(b)
    assert np.allclose(orc.matmul(a, b), want.numpy(), rtol=1e-5, atol=1e-5)
    b2 = rnd((2, 3, 7, 4), 6)
    assert np.allclose(orc.matmul(a, b2), (torch.from_numpy(a) @ torch.from_numpy(b2)).numpy(), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("name,fn", [
    ("gelu", F.gelu), ("silu", F.silu), ("sigmoid", torch.sigmoid), ("exp", torch.exp), ("neg", torch.neg),
    ("rsqrt", torch.rsqrt), ("sqrt", torch.sqrt), ("tanh", torch.tanh), ("erf", torch.erf), ("relu", torch.relu),
    ("abs", torch.abs), ("reciprocal", torch.reciprocal), ("log", torch.log), ("sin", torch.sin), ("cos", torch.cos),
    ("floor", torch.floor), ("ceil", torch.ceil), ("sign", torch.sign), ("hardsigmoid", F.hardsigmoid), ("mish", F.mish),
    ("acos", torch.acos), ("asin", torch.asin), ("asinh", torch.asinh), ("log1p", torch.log1p),
    ("cbrt", lambda t: torch.sign(t) * torch.abs(t) ** (1.0 / 3.0))])
def test_unary_matches_torch(orc, name, fn):
    x = rnd((1000,), 7, 3.0)
    if name in ("rsqrt", "sqrt", "log", "log1p"):
        x = np.abs(x) + 0.01
    if name in ("acos", "asin"):
        x = np.tanh(x)
    want = fn(torch.from_numpy(x).double()).float().numpy()
    assert np.allclose(orc.unary(name, x), want, rtol=2e-6, atol=2e-7)


def test_remaining_unary_ops_match_torch_on_ordinary_and_special_values(orc):
    """tan / atan / erfc / expm1 / leaky_relu / relu6 / isfinite / logical_not against the torch routines the goldens call
    (tools/golden/mapping.py:3954-3971 leaky_relu, 2586-2605 and 5076-5079 logical_not, 5868-5872 isfinite), and every unary op
    on the values where a plausible mistake shows: both zeros, both infinities, NaN, the knees of the piecewise ops."""
    x = rnd((1000,), 27, 3.0)
    t = torch.from_numpy(x).double()
    for name, want in (("tan", torch.tan(t)), ("atan", torch.atan(t)), ("erfc", torch.erfc(t)), ("expm1", torch.expm1(t)),
                       ("relu6", F.relu6(t))):
        assert np.allclose(orc.unary(name, x), want.float().numpy(), rtol=3e-6, atol=2e-7), name
    for slope in (0.01, 0.2, -0.5):
        assert np.array_equal(orc.unary("leaky_relu", x, slope), F.leaky_relu(torch.from_numpy(x), negative_slope=slope).numpy())
    sp = np.array([0.0, -0.0, 1.0, -1.0, 6.0, 6.5, -3.0, 3.0, np.inf, -np.inf, np.nan, 1e-30, -1e-30], dtype=np.float32)
    ts = torch.from_numpy(sp)
    assert np.array_equal(orc.unary("isfinite", sp), torch.isfinite(ts).float().numpy())
    assert np.array_equal(orc.unary("logical_not", sp), torch.logical_not(ts).float().numpy())   # NaN and the infinities are true
    fns = dict(abs=torch.abs, neg=torch.neg, relu=torch.relu, relu6=F.relu6, sign=torch.sign, floor=torch.floor, ceil=torch.ceil,
               sigmoid=torch.sigmoid, silu=F.silu, gelu=F.gelu, tanh=torch.tanh, erf=torch.erf, erfc=torch.erfc, exp=torch.exp,
               expm1=torch.expm1, atan=torch.atan, hardsigmoid=F.hardsigmoid, sqrt=torch.sqrt, rsqrt=torch.rsqrt,
               reciprocal=torch.reciprocal, log=torch.log, log1p=torch.log1p, asinh=torch.asinh)
    for name, fn in fns.items():
        got, want = orc.unary(name, sp), fn(ts.double()).float().numpy()   # in double: torch's own fp32 gelu is off by 1e-4 at -3
        assert np.allclose(got, want, rtol=1e-5, atol=1e-37, equal_nan=True), (name, got, want)
        both = np.isfinite(got) & (got == 0)
        # relu(-0.0): +0.0 like arith.maximumf of the reference's CPU lowering, where torch.relu keeps -0.0
        if name != "relu":
            assert np.array_equal(np.signbit(got[both]), np.signbit(want[both])), (name, got, want)


def test_comparison_binaries_match_numpy_including_nan(orc):
    a = np.array([[1.0, 2.0, np.nan, -0.0, np.inf, 3.0]], dtype=np.float32)
    b = np.array([[1.0], [3.0], [np.nan], [0.0], [np.inf], [-np.inf]], dtype=np.float32)
    with np.errstate(invalid="ignore"):
        for name, fn in (("eq", np.equal), ("ne", np.not_equal), ("ge", np.greater_equal), ("gt", np.greater), ("le", np.less_equal),
                         ("lt", np.less)):
            assert np.array_equal(orc.binary(name, a, b), fn(a, b).astype(np.float32)), name


def test_gelu_doc_example(orc):
    # include/ttmlir/Dialect/TTIR/IR/TTIROps.td:529-537: gelu([1, -1, 0...]) -> [0.8413, -0.1587, 0]
    y = orc.unary("gelu", np.array([1.0, -1.0, 0.0], dtype=np.float32))
    assert np.allclose(y, [0.8413447, -0.1586553, 0.0], atol=1e-6)


def test_binary_broadcast(orc):
    a, b = rnd((2, 1, 5, 7), 8), rnd((3, 1, 7), 9)
    for name, fn in (("add", np.add), ("multiply", np.multiply), ("subtract", np.subtract), ("divide", np.divide)):
        assert np.array_equal(orc.binary(name, a, b), fn(a, b))
    assert np.array_equal(orc.binary("gt", a, b), (a > b).astype(np.float32))


def test_rms_norm_matches_torch(orc):
    x, w, b = rnd((6, 40), 10), rnd((40,), 11), rnd((40,), 12)
    want = F.rms_norm(torch.from_numpy(x), (40,), torch.from_numpy(w), 1e-5) + torch.from_numpy(b)
    assert np.allclose(orc.rms_norm(x, w, b, 1e-5), want.numpy(), rtol=1e-5, atol=1e-6)
    # closed form: a constant row c normalises to c / sqrt(c^2 + eps)
    c = np.full((1, 16), 3.0, dtype=np.float32)
    assert np.allclose(orc.rms_norm(c, None, None, 0.0), 1.0)
    # eps matters: a dropped eps would turn an all-zero row into NaN
    assert np.array_equal(orc.rms_norm(np.zeros((1, 8), np.float32), None, None, 1e-5), np.zeros((1, 8), np.float32))


def test_softmax_and_reduce(orc):
    x = rnd((3, 5, 17), 13, 4.0)
    for dim in (-1, 1, 0):
        want = F.softmax(torch.from_numpy(x).double(), dim=dim).float().numpy()
        got = orc.softmax(x, dim)
        assert np.allclose(got, want, rtol=1e-5, atol=1e-7)
        assert np.allclose(got.sum(axis=dim), 1.0, atol=1e-5)
    big = np.array([[1000.0, 1000.0, -1000.0]], dtype=np.float32)        # max subtraction keeps this finite
    assert np.allclose(orc.softmax(big), [[0.5, 0.5, 0.0]])
    for op, fn in (("sum", np.sum), ("mean", np.mean), ("max", np.max), ("min", np.min)):
        for dim in (-1, 0, 1):
            assert np.allclose(orc.reduce(op, x, dim), fn(x.astype(np.float64), axis=dim), rtol=1e-5, atol=1e-5)
    assert orc.reduce("sum", x, -1, keepdim=True).shape == (3, 5, 1)


def test_rowwise_ops_on_special_values_match_torch(orc):
    """NaN, infinities and signed zeros through the reductions, softmax, RMSNorm and argmax: a NaN anywhere in a row makes
    max and min NaN (torch.max / torch.min, tools/golden/mapping.py:5189-5220, 2815-2856), a row of -inf gives a NaN softmax,
    the first NaN wins argmax."""
    x = np.array([[1.0, np.nan, 3.0, -2.0], [np.inf, 1.0, 2.0, 0.0], [-np.inf, -np.inf, 1.0, 0.0], [-np.inf] * 4,
                  [np.inf, np.inf, 0.0, 0.0], [0.0, -0.0, 0.0, -0.0], [5.0, 4.0, np.nan, np.nan]], dtype=np.float32)
    t = torch.from_numpy(x)
    for op, fn in (("sum", lambda t: t.sum(-1)), ("mean", lambda t: t.mean(-1)), ("max", lambda t: t.max(-1).values),
                   ("min", lambda t: t.min(-1).values)):
        assert np.array_equal(orc.reduce(op, x, -1), fn(t).numpy(), equal_nan=True), op
        assert np.array_equal(orc.reduce(op, x.T.copy(), 0), fn(t).numpy(), equal_nan=True), op
    assert np.allclose(orc.softmax(x, -1), F.softmax(t, -1).numpy(), rtol=1e-6, equal_nan=True)
    assert np.array_equal(orc.rms_norm(x, None, None, 1e-5), F.rms_norm(t, (4,), None, 1e-5).numpy(), equal_nan=True)
    assert np.array_equal(orc.argmax(x, -1), t.argmax(-1).numpy())


@pytest.mark.parametrize("causal", [False, True])
def test_sdpa_matches_torch(orc, causal):
    B, Hq, Hkv, S, D = 2, 4, 2, 24, 16
    q, k, v = rnd((B, Hq, S, D), 14), rnd((B, Hkv, S, D), 15), rnd((B, Hkv, S, D), 16)
    kr = torch.from_numpy(k).repeat_interleave(Hq // Hkv, dim=1)
    vr = torch.from_numpy(v).repeat_interleave(Hq // Hkv, dim=1)
    want = F.scaled_dot_product_attention(torch.from_numpy(q), kr, vr, is_causal=causal)
    assert np.allclose(orc.sdpa(q, k, v, is_causal=causal), want.numpy(), rtol=1e-4, atol=1e-5)
    if not causal:
        mask = rnd((B, 1, S, S), 17)
        want = F.scaled_dot_product_attention(torch.from_numpy(q), kr, vr, attn_mask=torch.from_numpy(mask), scale=0.3)
        assert np.allclose(orc.sdpa(q, k, v, mask=mask, scale=0.3), want.numpy(), rtol=1e-4, atol=1e-5)


def test_sdpa_uniform_keys_average_values(orc):
    # q = 0 -> uniform attention: causal row i is the mean of v[0..i]
    q = np.zeros((1, 1, 4, 8), np.float32)
    k = rnd((1, 1, 4, 8), 18)
    v = rnd((1, 1, 4, 8), 19)
    out = orc.sdpa(q, k, v, is_causal=True)[0, 0]
    for i in range(4):
        assert np.allclose(out[i], v[0, 0, : i + 1].mean(axis=0), atol=1e-6)


def test_pcc_special_cases():
    import oracle.metrics as m
    a = np.array([1.0, 2.0, 3.0, 4.0])
    assert m.get_pcc(a, a) == 1.0
    assert abs(m.get_pcc(a, 2 * a + 1) - 1.0) < 1e-12
    assert abs(m.get_pcc(a, -a) + 1.0) < 1e-12
    assert m.get_pcc(np.zeros(4), np.ones(4)) == 0.0                 # any-nonzero mismatch
    assert m.get_pcc(np.full(4, np.nan), np.full(4, np.nan)) == 1.0
    assert m.get_pcc(np.full(4, 2.0), np.full(4, 2.0 + 1e-9)) == 1.0  # two constants -> isclose
    assert m.get_pcc(np.zeros((0,)), np.zeros((0,))) == 1.0
    assert m.get_pcc(np.array([3.0]), np.array([3.1])) == 1.0         # single non-zero golden: cosine sign
    x = np.random.default_rng(0).standard_normal(1000)
    y = x + 0.1 * np.random.default_rng(1).standard_normal(1000)
    assert abs(m.get_pcc(x, y) - np.corrcoef(x, y)[0, 1]) < 1e-12
    at, rt = m.get_atol_rtol(np.array([1.0, 2.0]), np.array([1.5, 2.0]))
    assert at == 0.5 and abs(rt - 0.5 / 1.5) < 1e-12


# ---- decode path
def test_rotary_embedding_is_a_plane_rotation(orc):
    # pair (x[d], x[d + D/2]) with cos = cos(t), sin = sin(t) is the complex product (x1 + i x2) e^{it}
    B, S, D = 3, 5, 16
    x = rnd((B, S, D), 30)
    theta = np.random.default_rng(31).uniform(-3, 3, (S, D // 2)).astype(np.float32)
    cos = np.concatenate([np.cos(theta), np.cos(theta)], axis=-1)
    sin = np.concatenate([np.sin(theta), np.sin(theta)], axis=-1)
    out = orc.rotary_embedding(x, cos, sin)
    z = (x[..., : D // 2].astype(np.complex128) + 1j * x[..., D // 2:]) * np.exp(1j * theta.astype(np.float64))
    assert np.allclose(out[..., : D // 2], z.real, atol=1e-5) and np.allclose(out[..., D // 2:], z.imag, atol=1e-5)
    # special cases: cos = 1, sin = 0 is the identity; cos = 0, sin = 1 is rotate_half itself
    one, zero = np.ones((S, D), np.float32), np.zeros((S, D), np.float32)
    assert np.array_equal(orc.rotary_embedding(x, one, zero), x)
    rh = orc.rotary_embedding(x, zero, one)
    assert np.array_equal(rh[..., : D // 2], -x[..., D // 2:]) and np.array_equal(rh[..., D // 2:], x[..., : D // 2])
    # decode mode: every row uses the cache row named by token_index
    t3 = orc.rotary_embedding(x, cos, sin, token_index=3)
    assert np.allclose(t3[:, 0], orc.rotary_embedding(x[:, :1], cos[3:4], sin[3:4])[:, 0], atol=0)
    assert np.allclose(t3[:, 4], orc.rotary_embedding(x[:, 4:5], cos[3:4], sin[3:4])[:, 0], atol=0)


def test_cache_update_and_fill_match_slice_assignment(orc):
    U, H, S, D, Bin = 4, 3, 64, 8, 2
    cache = rnd((U, H, S, D), 32)
    upd = rnd((1, H, Bin, D), 33)
    got = orc.update_cache(cache, upd, 37, batch_offset=1)
    want = torch.from_numpy(cache.copy())
    want[1:3, :, 37, :] = torch.from_numpy(upd)[0].permute(1, 0, 2)      # tools/golden/mapping.py:3664-3671
    assert np.array_equal(got, want.numpy())
    assert np.array_equal(orc.update_cache(cache, upd[:, :, :1], 0)[0, :, 0], upd[0, :, 0])
    fill = rnd((1, H, 40, D), 34)
    got = orc.fill_cache(cache, fill, batch_offset=2)
    want = cache.copy()
    want[2, :, :40] = fill[0]
    want[2, :, 40:64] = 0                                                  # rows up to the tile boundary are cleared
    assert np.array_equal(got, want)
    assert np.array_equal(orc.fill_cache(cache, fill[:, :, :32])[0, :, 32:], cache[0, :, 32:])   # aligned: nothing cleared


def test_paged_cache_writes_by_hand_and_against_the_unpaged_ops(orc):
    """Known answers written out cell by cell for a 2-user page table, then the relation that ties the paged ops to the
    unpaged ones: with the identity page table (page p of user u is block u * pages + p) a paged cache is the unpaged
    cache [users, heads, pages * block, dim] viewed block-wise, so both routes must leave the same bytes."""
    blocks, H, bs, D = 5, 2, 32, 8
    cache = rnd((blocks, H, bs, D), 40)
    inp = rnd((1, 2, H, D), 41)
    table = np.array([[2, 0], [1, 3]], dtype=np.int32)
    got = orc.paged_update_cache(cache, inp, np.array([33, 5]), table)
    want = cache.copy()
    want[0, :, 1, :] = inp[0, 0]        # user 0, position 33 = second page (block 0), offset 1
    want[1, :, 5, :] = inp[0, 1]        # user 1, position 5 = first page (block 1), offset 5
    assert np.array_equal(got, want)
    # positions past the table, negative positions and block numbers outside the cache write nothing
    assert np.array_equal(orc.paged_update_cache(cache, inp, np.array([64, -1]), table), cache)
    assert np.array_equal(orc.paged_update_cache(cache, inp, np.array([0, 0]), np.array([[7, 0], [-2, 3]], dtype=np.int32)), cache)
    # static cache: user u owns entry u, or entry 0 for everyone when shared (the last user wins)
    got = orc.paged_update_cache(cache, inp, np.array([3, 9]))
    want = cache.copy()
    want[0, :, 3, :], want[1, :, 9, :] = inp[0, 0], inp[0, 1]
    assert np.array_equal(got, want)
    got = orc.paged_update_cache(cache, inp, np.array([3, 3]), share_cache=True)
    assert np.array_equal(got[0, :, 3, :], inp[0, 1]) and np.array_equal(got[1:], cache[1:])
    # fill: 40 positions of one sequence through row 1 of the table: 32 rows into block 1, 8 into block 3
    fill = rnd((1, H, 40, D), 42)
    got = orc.paged_fill_cache(cache, fill, table, batch_idx=np.array([1]))
    want = cache.copy()
    want[1] = fill[0, :, :32]
    want[3, :, :8] = fill[0, :, 32:]
    assert np.array_equal(got, want)
    # identity page table against the unpaged ops
    users, pages = 3, 2
    flat = rnd((users, H, pages * bs, D), 43)
    paged = flat.reshape(users, H, pages, bs, D).transpose(0, 2, 1, 3, 4).reshape(users * pages, H, bs, D).copy()
    ident = np.arange(users * pages, dtype=np.int32).reshape(users, pages)
    back = lambda c: c.reshape(users, pages, H, bs, D).transpose(0, 2, 1, 3, 4).reshape(users, H, pages * bs, D)
    seq = rnd((1, H, 2 * bs, D), 44)
    assert np.array_equal(back(orc.paged_fill_cache(paged, seq, ident, batch_idx=np.array([2]))), orc.fill_cache(flat, seq, batch_offset=2))
    step = rnd((1, users, H, D), 45)
    same_pos = orc.update_cache(flat, np.ascontiguousarray(step.transpose(0, 2, 1, 3)), 45)
    assert np.array_equal(back(orc.paged_update_cache(paged, step, np.array([45, 45, 45]), ident)), same_pos)


@pytest.mark.parametrize("H,Hkv", [(4, 4), (8, 2)])
def test_sdpa_decode_against_library_attention(orc, H, Hkv):
    B, S, D = 3, 48, 16
    q, k, v = rnd((1, B, H, D), 35), rnd((B, Hkv, S, D), 36), rnd((B, Hkv, S, D), 37)
    cur = np.array([0, 17, 47], np.int32)
    got = orc.sdpa_decode(q, k, v, cur_pos=cur)
    qt = torch.from_numpy(q)[0].unsqueeze(2)                               # [B, H, 1, D]
    kr = torch.from_numpy(k).repeat_interleave(H // Hkv, dim=1)
    vr = torch.from_numpy(v).repeat_interleave(H // Hkv, dim=1)
    keep = (torch.arange(S)[None, :] <= torch.from_numpy(cur).long()[:, None])[:, None, None, :]
    want = F.scaled_dot_product_attention(qt, kr, vr, attn_mask=keep).squeeze(2).unsqueeze(0)
    assert np.allclose(got, want.numpy(), rtol=1e-4, atol=1e-5)
    # the prefill oracle with one query row per head agrees when nothing is masked
    full = orc.sdpa(np.ascontiguousarray(qt.numpy()), k, v)
    assert np.allclose(orc.sdpa_decode(q, k, v, is_causal=False)[0], full[:, :, 0], rtol=1e-5, atol=1e-6)
    # additive mask enters before the scale: (q k + m) * s
    m = rnd((B, 1, H, S), 38)
    got = orc.sdpa_decode(q, k, v, mask=m, scale=0.25)
    want = F.scaled_dot_product_attention(qt, kr, vr, attn_mask=torch.from_numpy(m).permute(0, 2, 1, 3) * 0.25, scale=0.25)
    assert np.allclose(got[0], want.squeeze(2).numpy(), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
def test_sdpa_sliding_window_against_library_attention_with_a_band_mask(orc, causal):
    """The window restated through torch's attention with a boolean band (tools/golden/mapping.py:8450-8467 gives the
    band's edges), plus the cases the band's definition fixes without any formula: a causal window as long as the
    sequence is plain causal attention, a causal window of one key returns the value rows themselves, a symmetric
    window of width 0 (or 1: half = 0) does too."""
    B, Hq, Hkv, S, D = 2, 4, 2, 40, 16
    q, k, v = rnd((B, Hq, S, D), 40), rnd((B, Hkv, S, D), 41), rnd((B, Hkv, S, D), 42)
    kr = torch.from_numpy(k).repeat_interleave(Hq // Hkv, dim=1)
    vr = torch.from_numpy(v).repeat_interleave(Hq // Hkv, dim=1)
    i, j = torch.arange(S)[:, None], torch.arange(S)[None, :]
    for w in (1, 2, 7, 16, 39, 40, 100):
        keep = ((i - j >= 0) & (i - j < w)) if causal else ((i - j).abs() <= w // 2)
        want = F.scaled_dot_product_attention(torch.from_numpy(q), kr, vr, attn_mask=keep)
        got = orc.sdpa(q, k, v, is_causal=causal, sliding_window=w)
        assert np.allclose(got, want.numpy(), rtol=1e-4, atol=1e-5), w
    if causal:
        assert np.array_equal(orc.sdpa(q, k, v, is_causal=True, sliding_window=S), orc.sdpa(q, k, v, is_causal=True))
        assert np.allclose(orc.sdpa(q, k, v, is_causal=True, sliding_window=1), vr.numpy(), atol=1e-6)
    else:
        assert np.array_equal(orc.sdpa(q, k, v, sliding_window=2 * S), orc.sdpa(q, k, v))
        for w in (0, 1):
            assert np.allclose(orc.sdpa(q, k, v, sliding_window=w), vr.numpy(), atol=1e-6)
    # a mask given as well is added on top of the window
    m = rnd((B, 1, S, S), 43)
    keep = ((i - j >= 0) & (i - j < 5)) if causal else ((i - j).abs() <= 2)
    want = F.scaled_dot_product_attention(torch.from_numpy(q), kr, vr,
                                          attn_mask=torch.from_numpy(m).masked_fill(~keep, float("-inf")))
    # (a causal op carries no mask in the reference; the oracle adds one all the same)
    assert np.allclose(orc.sdpa(q, k, v, mask=m, is_causal=causal, sliding_window=5), want.numpy(), rtol=1e-4, atol=1e-5)


def test_sdpa_attention_sink_is_one_more_key_with_a_zero_value_row(orc):
    """The sink as the golden has it (tools/golden/mapping.py:8476-8494: a column concatenated to the scores before the
    softmax and dropped after it) is attention over one more key whose value row is zero.  With the last coordinate of
    every query fixed at 1 and of every real key at 0, the extra key (0, ..., 0, x_h / scale) has the logit x_h for every
    query of head h: the plain oracle on the extended tensors must equal the oracle with the sink operand x_h / scale
    (the operand is the logit divided by the scale, lib/Conversion/TTIRToTTNN/TTIRToTTNN.cpp:3507-3533)."""
    B, H, Sq, Sk, D = 2, 3, 9, 12, 8
    q, k, v = rnd((B, H, Sq, D), 44), rnd((B, H, Sk, D), 45), rnd((B, H, Sk, D), 46)
    q[..., -1] = 1.0
    k[..., -1] = 0.0
    x = np.array([-1.5, 0.0, 2.25], np.float32)                  # logits per head
    for scale in (None, 0.5, 1.0):
        s = scale if scale else 1.0 / np.sqrt(D)
        k_ext = np.concatenate([k, np.zeros((B, H, 1, D), np.float32)], axis=2)
        k_ext[:, :, -1, -1] = (x / s)[None, :]
        v_ext = np.concatenate([v, np.zeros((B, H, 1, D), np.float32)], axis=2)
        want = orc.sdpa(q, k_ext, v_ext, scale=scale)
        got = orc.sdpa(q, k, v, scale=scale, attention_sink=(x / s).reshape(1, H, 1, 1))
        assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
        assert not np.allclose(got, orc.sdpa(q, k, v, scale=scale), atol=1e-3)
    # a sink far below every score changes nothing, one far above takes all the weight
    assert np.allclose(orc.sdpa(q, k, v, attention_sink=np.full(H, -1e4, np.float32)), orc.sdpa(q, k, v), atol=1e-6)
    assert np.max(np.abs(orc.sdpa(q, k, v, attention_sink=np.full(H, 1e4, np.float32)))) < 1e-6
    # grouped heads: the sink is per QUERY head
    kg, vg = k[:, :1], v[:, :1]
    got = orc.sdpa(q, kg, vg, attention_sink=x)
    for h in range(H):
        one = orc.sdpa(q[:, h:h + 1], kg, vg, attention_sink=x[h:h + 1])
        assert np.array_equal(got[:, h:h + 1], one)
    # causal + window + sink together, against the extended-key form with the band written as a mask
    S = 9
    q2, k2, v2 = q[:, :, :S], k[:, :, :S], v[:, :, :S]
    i, j = np.arange(S)[:, None], np.arange(S)[None, :]
    band = np.where((i - j >= 0) & (i - j < 4), 0.0, -np.inf).astype(np.float32)
    band_ext = np.concatenate([band, np.zeros((S, 1), np.float32)], axis=1)[None, None]
    s = 1.0 / np.sqrt(D)
    k_ext = np.concatenate([k2, np.zeros((B, H, 1, D), np.float32)], axis=2)
    k_ext[:, :, -1, -1] = (x / s)[None, :]
    v_ext = np.concatenate([v2, np.zeros((B, H, 1, D), np.float32)], axis=2)
    want = orc.sdpa(q2, k_ext, v_ext, mask=np.broadcast_to(band_ext, (B, 1, S, S + 1)))
    got = orc.sdpa(q2, k2, v2, is_causal=True, sliding_window=4, attention_sink=x / s)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6)


def test_sdpa_decode_window_and_sink(orc):
    """Decode: the window keeps keys [max(0, p - w + 1), p] (tools/golden/mapping.py:8814-8824), checked against torch's
    attention with that set written as a boolean mask, and against the prefill oracle's last causal row; the sink against
    a cache that holds the extra key at position 0 (k = 0 -> logit 0, v = 0) with every position shifted by one."""
    B, H, Hkv, S, D = 3, 4, 2, 64, 16
    q, k, v = rnd((1, B, H, D), 47), rnd((B, Hkv, S, D), 48), rnd((B, Hkv, S, D), 49)
    cur = np.array([3, 30, 63], np.int32)
    qt = torch.from_numpy(q)[0].unsqueeze(2)
    kr = torch.from_numpy(k).repeat_interleave(H // Hkv, dim=1)
    vr = torch.from_numpy(v).repeat_interleave(H // Hkv, dim=1)
    j, p = torch.arange(S)[None, :], torch.from_numpy(cur).long()[:, None]
    for w in (1, 4, 17, 31, 64, 200):
        keep = ((j <= p) & (j >= p - w + 1))[:, None, None, :]
        want = F.scaled_dot_product_attention(qt, kr, vr, attn_mask=keep).squeeze(2).unsqueeze(0)
        assert np.allclose(orc.sdpa_decode(q, k, v, cur_pos=cur, sliding_window=w), want.numpy(), rtol=1e-4, atol=1e-5), w
    assert np.array_equal(orc.sdpa_decode(q, k, v, cur_pos=cur, sliding_window=S), orc.sdpa_decode(q, k, v, cur_pos=cur))
    # window of one key: the value row at the decode position
    one = orc.sdpa_decode(q, k, v, cur_pos=cur, sliding_window=1)
    for b in range(B):
        assert np.allclose(one[0, b], vr[b, :, cur[b]].numpy(), atol=1e-6)
    # without cur_pos the window ends at the last position
    last = orc.sdpa_decode(q, k, v, cur_pos=np.full(B, S - 1, np.int32), sliding_window=9)
    assert np.array_equal(orc.sdpa_decode(q, k, v, is_causal=False, sliding_window=9), last)
    # the decode of user b at position p is row p of causal windowed prefill attention over the same keys
    qrow = np.zeros((1, H, S, D), np.float32)
    qrow[0, :, 30] = q[0, 1]
    pre = orc.sdpa(qrow, k[1:2], v[1:2], is_causal=True, sliding_window=17)
    assert np.allclose(orc.sdpa_decode(q, k, v, cur_pos=cur, sliding_window=17)[0, 1], pre[0, :, 30], rtol=1e-5, atol=1e-6)
    # sink with logit 0 = one more visible key with k = 0 and v = 0
    k_sh = np.concatenate([np.zeros((B, Hkv, 1, D), np.float32), k[:, :, :-1]], axis=2)
    v_sh = np.concatenate([np.zeros((B, Hkv, 1, D), np.float32), v[:, :, :-1]], axis=2)
    cur2 = np.array([3, 30, 62], np.int32)
    want = orc.sdpa_decode(q, k_sh, v_sh, cur_pos=cur2 + 1)
    got = orc.sdpa_decode(q, k, v, cur_pos=cur2, attention_sink=np.zeros((H, 32), np.float32))
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
    # the operand is multiplied by the scale like the scores: the same logits written for two scales give, with q
    # rescaled to keep q k scale fixed, the same output
    sink = np.tile(np.array([0.5, -2.0, 3.0, 1.0], np.float32)[:, None], (1, 32))
    a = orc.sdpa_decode(q, k, v, cur_pos=cur, scale=0.25, attention_sink=sink)
    b_ = orc.sdpa_decode(q * 0.5, k, v, cur_pos=cur, scale=0.5, attention_sink=sink * 0.5)
    assert np.allclose(a, b_, rtol=1e-5, atol=1e-6)
    assert not np.allclose(a, orc.sdpa_decode(q, k, v, cur_pos=cur, scale=0.25), atol=1e-3)
    # the decode sink agrees with the prefill oracle's (one query row, everything visible)
    full = orc.sdpa(np.ascontiguousarray(qt.numpy()), k, v, attention_sink=sink[:, 0])
    assert np.allclose(orc.sdpa_decode(q, k, v, is_causal=False, attention_sink=sink)[0], full[:, :, 0], rtol=1e-5, atol=1e-6)


def test_index_and_select_ops_against_torch(orc):
    """where / embedding / argmax / arange / repeat / maximum, minimum, remainder, pow, atan2: the oracle's numpy calls
    against the torch calls the reference's goldens make (tools/golden/mapping.py:2900-2912, 4259-4290, 4493-4570,
    5222-5265, 5516-5530, 5579-5586), including what differs between the libraries' conventions: ties and NaN in
    argmax, clamped indices, remainder's sign, NaN through maximum."""
    g = torch.Generator().manual_seed(50)
    c = (torch.rand((3, 1, 5), generator=g) > 0.5).float()
    a, b = torch.randn((3, 4, 5), generator=g), torch.randn((1, 4, 1), generator=g)
    assert np.array_equal(orc.where(c.numpy(), a.numpy(), b.numpy()), torch.where(c != 0, a, b).numpy())
    assert np.array_equal(orc.where(np.array([-0.0, 0.0, np.nan, 2.0]), np.ones(4), np.zeros(4)), np.array([0.0, 0.0, 1.0, 1.0]))
    w = torch.randn((1, 1, 11, 6), generator=g)
    idx = torch.tensor([[0, 10, 3], [25, -4, 7]])
    want = F.embedding(idx.clamp(0, 10), w.reshape(11, 6))
    assert np.array_equal(orc.embedding(idx.numpy(), w.numpy()), want.numpy())
    x = torch.randn((2, 3, 7), generator=g)
    x[0, 1, 2] = x[0, 1, 5] = 9.0                               # tie: the first index wins
    x[1, 2, 4] = float("nan")                                   # NaN counts as the largest value
    for dim in (0, 1, 2, -1):
        for keep in (False, True):
            assert np.array_equal(orc.argmax(x.numpy(), dim, keep), torch.argmax(x, dim=dim, keepdim=keep).numpy())
    assert int(orc.argmax(x.numpy())) == int(torch.argmax(x))
    assert orc.argmax(x.numpy(), keep_dim=True).shape == (1, 1, 1)
    for start, end, step in ((0, 10, 1), (3, 40, 4), (5, -5, -2), (0, 1, 0.125)):
        assert np.array_equal(orc.arange(start, end, step), torch.arange(start, end, step, dtype=torch.float32).numpy())
    assert np.array_equal(orc.arange(0, 300, 1, np.int32), torch.arange(0, 300, 1, dtype=torch.float32).to(torch.int32).numpy())
    assert np.array_equal(orc.repeat(a.numpy(), (2, 1, 3)), a.repeat(2, 1, 3).numpy())
    p, q = torch.randn((4, 6), generator=g) * 3, torch.randn((1, 6), generator=g) * 2
    p[0, 0] = float("nan")
    for name, fn in (("maximum", torch.maximum), ("minimum", torch.minimum), ("remainder", torch.remainder), ("atan2", torch.atan2)):
        assert np.allclose(orc.binary_composite(name, p.numpy(), q.numpy()), fn(p, q.expand(4, 6)).numpy(), rtol=1e-6, atol=1e-6, equal_nan=True), name
    assert np.allclose(orc.binary_composite("pow", p.abs().numpy(), q.numpy()), torch.pow(p.abs(), q).numpy(), rtol=1e-5, equal_nan=True)
    assert orc.binary_composite("remainder", np.float32(-7), np.float32(3)) == 2.0 and orc.binary_composite("remainder", np.float32(7), np.float32(-3)) == -2.0


def test_clamp_against_torch(orc):
    x = rnd((500,), 51, 4.0)
    x[:3] = [np.nan, np.inf, -np.inf]
    for lo, hi in ((-1.0, 2.5), (0.0, 0.0), (-3.0, -1.0)):
        assert np.array_equal(orc.clamp(x, lo, hi), torch.clamp(torch.from_numpy(x), min=lo, max=hi).numpy(), equal_nan=True)


def test_chunked_sdpa_is_causal_attention_of_the_chunk_over_the_unpaged_prefix(orc):
    """tools/golden/mapping.py:8847-8913 builds the same thing from torch: unpage with the table, mask col <= start + row,
    F.scaled_dot_product_attention.  Also fixed by the definition: a chunk that starts at 0 and spans the cache is plain
    causal attention, and the rows of a later chunk are the last rows of the causal attention over the whole sequence."""
    rng = np.random.default_rng(7)
    B, H, Hkv, Sq, D, block, pages = 2, 4, 2, 40, 32, 32, 4
    Sk = block * pages
    k = rng.standard_normal((B, Hkv, Sk, D)).astype(np.float32)
    v = rng.standard_normal((B, Hkv, Sk, D)).astype(np.float32)
    table = rng.permutation(B * pages).reshape(B, pages)
    kp = np.zeros((B * pages, Hkv, block, D), np.float32)
    vp = np.zeros_like(kp)
    for b in range(B):
        for p in range(pages):
            kp[table[b, p]] = k[b, :, p * block:(p + 1) * block]
            vp[table[b, p]] = v[b, :, p * block:(p + 1) * block]
    for start in (0, 17, Sk - Sq):
        q = rng.standard_normal((B, H, Sq, D)).astype(np.float32)
        got = orc.chunked_sdpa(q, kp, vp, table, start)
        col, row = torch.arange(Sk).view(1, Sk), (start + torch.arange(Sq)).view(Sq, 1)
        m = torch.zeros((1, 1, Sq, Sk)).masked_fill_(~(col <= row).view(1, 1, Sq, Sk), torch.finfo(torch.float32).min)
        rep = lambda t: torch.repeat_interleave(torch.from_numpy(t), H // Hkv, dim=1)
        want = F.scaled_dot_product_attention(torch.from_numpy(q), rep(k), rep(v), attn_mask=m).numpy()
        assert np.max(np.abs(got - want)) <= 2e-6
    # the last Sq rows of plain causal attention over all Sk positions
    qfull = rng.standard_normal((B, H, Sk, D)).astype(np.float32)
    full = orc.sdpa(qfull, k, v, is_causal=True)
    assert np.max(np.abs(orc.chunked_sdpa(qfull[:, :, Sk - Sq:], kp, vp, table, Sk - Sq) - full[:, :, Sk - Sq:])) <= 2e-6


def test_rotary_embedding_llama_with_the_pair_rotation_matrix_is_interleaved_rope(orc):
    """No golden exists for the op; what fixes it: with the matrix that maps (x[2i], x[2i+1]) to (-x[2i+1], x[2i]) - the one
    Llama passes - the result is the rotation of every interleaved pair by its angle; with the zero matrix it is x * cos;
    with the identity it is x * (cos + sin)."""
    rng = np.random.default_rng(8)
    x = rng.standard_normal((1, 3, 40, 64)).astype(np.float32)
    ang = rng.standard_normal((1, 1, 40, 32)).astype(np.float32)
    cos, sin = np.repeat(np.cos(ang), 2, -1), np.repeat(np.sin(ang), 2, -1)
    T = np.zeros((32, 32), np.float32)
    for i in range(16):
        T[2 * i + 1, 2 * i] = -1.0     # (x T)[2i] = -x[2i+1]
        T[2 * i, 2 * i + 1] = 1.0      # (x T)[2i+1] = x[2i]
    got = orc.rotary_embedding_llama(x, cos, sin, T)
    z = (x[..., 0::2] + 1j * x[..., 1::2]) * np.exp(1j * ang)
    want = np.stack([z.real, z.imag], -1).reshape(x.shape)
    assert np.max(np.abs(got - want)) <= 1e-5
    assert np.array_equal(orc.rotary_embedding_llama(x, cos, sin, np.zeros((32, 32))), x * cos)
    assert np.allclose(orc.rotary_embedding_llama(x, cos, sin, np.eye(32)), x * cos + x * sin, atol=1e-6)
