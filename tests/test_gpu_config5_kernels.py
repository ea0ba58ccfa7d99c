"""The launches of config 5 (Llama-3-8B decoder layer, 2048 tokens, hidden 4096, 32 / 8 heads of 128, FFN 14336) one by one,
at their real shapes and through the entry points the op runners call for that program: grouped Q / K / V projection, attention
on heads-inner operands, output projection with the residual add in its epilogue, RMSNorm, gate projection with SiLU, up
projection with the multiply in its epilogue, bfp4_b down projection with the residual add.  Each is compared with the oracle
on that launch's own inputs, so the bars are per-op bars: a result is the oracle's bf16 value or, where the fp32 value sits at a
rounding tie, its neighbour.  Linear launches are checked on 160 rows spread over the sequence (first and last tile rows
included), attention and RMSNorm on every output.  The whole program end to end is tests/test_gpu_runtime.py's job."""
import ctypes

import numpy as np
import pytest
import torch

from ttmlir_amd import datagen
from test_gpu_linear import tilize_dev, untilize_dev, pack_weight

pytestmark = pytest.mark.gpu

S, HID, NQ, NKV, HD, FFN = 2048, 4096, 32, 8, 128, 14336
ROWS = np.unique(np.concatenate([np.arange(0, 32), np.arange(2016, 2048), np.arange(37, 2048, 21)]))[:160]


@pytest.fixture(scope="module")
def metrics():
    import oracle.metrics as m
    return m


@pytest.fixture(scope="module", autouse=True)
def all_cores(orc):
    orc.set_threads(orc.max_threads())
    yield
    orc.set_threads(1)


def spacing(got, want):
    mag = np.maximum(np.maximum(np.abs(got), np.abs(want)), 2.0 ** -120)
    return np.exp2(np.floor(np.log2(mag)) - 7)


def assert_per_op_bar(metrics, got, want_f32, name, exact=0.995):
    """got: bf16 values from the GPU (as f32); want_f32: the oracle's f32 result before its cast back to bf16."""
    want = np.asarray(want_f32, dtype=np.float32)
    import oracle.oracle as orc
    wr = orc.round_bf16(want)
    err = np.abs(got - wr)
    sp = spacing(got, wr)
    frac = float(np.mean(got == wr))
    print("%s: max-abs %.5f, exact %.5f, worst err/spacing %.2f, pcc %.7f" % (name, err.max(), frac, (err / sp).max(),
                                                                              metrics.get_pcc(wr, got)), flush=True)
    assert np.all(np.isfinite(got))
    # the neighbour is allowed only where the fp32 value is within 2^-10 relative (+ 1e-4 absolute for sums that cancel) of
    # the midpoint; in terms of the rounded values: one spacing at most
    assert np.all(err <= sp + 1e-4), name
    assert frac >= exact, (name, frac)
    assert metrics.get_pcc(wr, got) >= 0.9999


def dequant(hip, dev, packed, fmt, K, N):
    back = torch.empty((K, N), dtype=torch.float32, device=dev)
    hip.call("ttm_bfp_unpack", hip.ptr(packed), fmt, hip.ptr(back), hip.F32, hip.ROW_MAJOR, 1, K, N, hip.current_stream())
    torch.cuda.synchronize()
    return back.cpu().numpy()


def test_rms_norm_2048x4096(hip, dev, orc, metrics):
    x = datagen.randn((S, HID), seed=300, dtype=torch.bfloat16)
    w = (1.0 + 0.02 * datagen.randn((HID,), seed=301)).to(torch.bfloat16)
    xt, wt = tilize_dev(hip, x, dev), tilize_dev(hip, w.reshape(1, -1), dev)
    out = torch.full_like(xt, float("nan"))
    hip.call("ttm_rms_norm", hip.ptr(xt), hip.ptr(wt), hip.TILE, None, hip.TILE, hip.ptr(out), hip.BF16, 1, S, HID, 1e-5,
             hip.current_stream())
    got = untilize_dev(hip, out, (S, HID), dev).float().cpu().numpy()
    assert_per_op_bar(metrics, got, orc.rms_norm(x.float().numpy(), w.float().numpy(), None, 1e-5), "rms_norm")


def test_grouped_qkv_projection(hip, dev, orc, metrics):
    """One ttm_linear_group launch for [2048, 4096] x bfp8_b {[4096, 4096], [4096, 1024], [4096, 1024]}."""
    a = datagen.randn((S, HID), seed=310, dtype=torch.bfloat16)
    Ns = (NQ * HD, NKV * HD, NKV * HD)
    ws = [datagen.randn((HID, N), seed=311 + i, std=0.02) for i, N in enumerate(Ns)]
    at = tilize_dev(hip, a, dev)
    wt = [pack_weight(hip, w, hip.BFP8B, dev) for w in ws]
    outs = [torch.full((S * N,), float("nan"), dtype=torch.bfloat16, device=dev) for N in Ns]
    n = len(Ns)
    wp = (ctypes.c_void_p * n)(*[t.data_ptr() for t in wt])
    op = (ctypes.c_void_p * n)(*[t.data_ptr() for t in outs])
    nn = (ctypes.c_int64 * n)(*Ns)
    hip.call("ttm_linear_group", hip.ptr(at), n, wp, hip.BFP8B, op, nn, None, S, HID, hip.current_stream())
    arows = a.float().numpy()[ROWS]
    for name, o, t, N in zip("qkv", outs, wt, Ns):
        got = untilize_dev(hip, o, (S, N), dev).float().cpu().numpy()[ROWS]
        assert_per_op_bar(metrics, got, orc.linear(arows, dequant(hip, dev, t, hip.BFP8B, HID, N)), "projection " + name)


def test_attention_on_heads_inner_operands(hip, dev, orc, metrics):
    """q [1, 2048, 32 * 128], k / v [1, 2048, 8 * 128] as the projections leave them, out [1, 2048, 32 * 128] as the output
    projection reads it (heads_inner = 15), causal, every output against the oracle."""
    q = datagen.randn((1, NQ, S, HD), seed=320, dtype=torch.bfloat16)
    k = datagen.randn((1, NKV, S, HD), seed=321, dtype=torch.bfloat16)
    v = datagen.randn((1, NKV, S, HD), seed=322, dtype=torch.bfloat16)
    inner = lambda t: t.permute(0, 2, 1, 3).reshape(1, S, t.shape[1] * HD).contiguous()
    qi, ki, vi = (tilize_dev(hip, inner(t), dev) for t in (q, k, v))
    out = torch.full_like(qi, float("nan"))
    hip.call("ttm_sdpa_heads_inner", hip.ptr(qi), hip.ptr(ki), hip.ptr(vi), None, 1, hip.ptr(out), hip.BF16, 1, NQ, NKV, S, S, HD, 1,
             0.0, 15, hip.current_stream())
    got = untilize_dev(hip, out, (1, S, NQ * HD), dev).float().cpu().numpy().reshape(1, S, NQ, HD).transpose(0, 2, 1, 3)
    want = orc.sdpa(q.float().numpy(), k.float().numpy(), v.float().numpy(), None, is_causal=True)
    err = np.abs(got - want)
    print("attention: max-abs %.5f, pcc %.7f" % (err.max(), metrics.get_pcc(want, got)), flush=True)
    # softmax numerators are rounded to bf16 before P.V (relative 2^-9 each, averaging out over the keys) and the output
    # once more: |out| < 4 -> half a spacing 2^-7, plus the numerators' share
    assert err.max() <= 2.0 ** -6
    assert metrics.get_pcc(want, got) >= 0.9999
    assert np.array_equal(got[0, :, 0, :], np.repeat(v.float().numpy()[0, :, 0, :], NQ // NKV, axis=0))   # one visible key


def linear_tail(hip, dev, a, wt, wfmt, N, act, tail_op, tail):
    M, K = a.shape
    at, tt = tilize_dev(hip, a, dev), (tilize_dev(hip, tail, dev) if tail is not None else None)
    out = torch.full((M * N,), float("nan"), dtype=torch.bfloat16, device=dev)
    hip.call("ttm_linear_tail", hip.ptr(at), hip.BF16, hip.ptr(wt), wfmt, 0, None, hip.BF16, hip.TILE, hip.ptr(out), hip.BF16, 1, 1,
             M, N, K, hip.ACT[act], tail_op, hip.ptr(tt) if tt is not None else None, hip.current_stream())
    return untilize_dev(hip, out, (M, N), dev).float().cpu().numpy()


def test_output_projection_with_residual_add(hip, dev, orc, metrics):
    a = datagen.randn((S, NQ * HD), seed=330, dtype=torch.bfloat16)
    x = datagen.randn((S, HID), seed=331, dtype=torch.bfloat16)
    wt = pack_weight(hip, datagen.randn((NQ * HD, HID), seed=332, std=0.02), hip.BFP8B, dev)
    got = linear_tail(hip, dev, a, wt, hip.BFP8B, HID, None, 1, x)[ROWS]
    o = orc.round_bf16(orc.linear(a.float().numpy()[ROWS], dequant(hip, dev, wt, hip.BFP8B, NQ * HD, HID)))
    want = orc.binary("add", o, x.float().numpy()[ROWS])
    # two roundings: the projection, then the sum.  Where the projection lands on the neighbour (one spacing of the
    # projection away), the sum moves by that much before its own rounding
    err = np.abs(got - orc.round_bf16(want))
    print("o projection + x: max-abs %.5f, exact %.5f" % (err.max(), np.mean(err == 0)), flush=True)
    assert np.all(err <= spacing(got, want) + spacing(o, o) + 1e-4) and np.mean(err == 0) >= 0.995
    assert metrics.get_pcc(orc.round_bf16(want), got) >= 0.9999


def test_gate_and_up_projections(hip, dev, orc, metrics):
    """SiLU(h Wg) by ttm_linear, then (h Wu) * gate in the up projection's epilogue: [2048, 4096] x bfp8_b [4096, 14336]."""
    h = datagen.randn((S, HID), seed=340, dtype=torch.bfloat16)
    wg = pack_weight(hip, datagen.randn((HID, FFN), seed=341, std=0.02), hip.BFP8B, dev)
    wu = pack_weight(hip, datagen.randn((HID, FFN), seed=342, std=0.02), hip.BFP8B, dev)
    gate = linear_tail(hip, dev, h, wg, hip.BFP8B, FFN, "silu", 0, None)
    hr = h.float().numpy()[ROWS]
    assert_per_op_bar(metrics, gate[ROWS], orc.linear(hr, dequant(hip, dev, wg, hip.BFP8B, HID, FFN), None, "silu"), "gate")
    prod = linear_tail(hip, dev, h, wu, hip.BFP8B, FFN, None, 2, torch.from_numpy(gate).to(torch.bfloat16))[ROWS]
    up = orc.round_bf16(orc.linear(hr, dequant(hip, dev, wu, hip.BFP8B, HID, FFN)))
    want = orc.binary("multiply", up, gate[ROWS])
    err = np.abs(prod - orc.round_bf16(want))
    print("up * gate: max-abs %.5f, exact %.5f" % (err.max(), np.mean(err == 0)), flush=True)
    # a neighbouring `up` moves the product by |gate| spacings of `up` before the product's own rounding
    assert np.all(err <= spacing(prod, want) + np.abs(gate[ROWS]) * spacing(up, up) + 1e-4) and np.mean(err == 0) >= 0.995


def test_down_projection_bfp4_with_residual_add(hip, dev, orc, metrics):
    m = datagen.randn((S, FFN), seed=350, dtype=torch.bfloat16)
    x = datagen.randn((S, HID), seed=351, dtype=torch.bfloat16)
    wt = pack_weight(hip, datagen.randn((FFN, HID), seed=352, std=0.02), hip.BFP4B, dev)
    got = linear_tail(hip, dev, m, wt, hip.BFP4B, HID, None, 1, x)[ROWS]
    d = orc.round_bf16(orc.linear(m.float().numpy()[ROWS], dequant(hip, dev, wt, hip.BFP4B, FFN, HID)))
    want = orc.binary("add", d, x.float().numpy()[ROWS])
    err = np.abs(got - orc.round_bf16(want))
    print("down projection + x: max-abs %.5f, exact %.5f" % (err.max(), np.mean(err == 0)), flush=True)
    assert np.all(err <= spacing(got, want) + spacing(d, d) + 1e-4) and np.mean(err == 0) >= 0.995
    assert metrics.get_pcc(orc.round_bf16(want), got) >= 0.9999
