"""The entry point that allocates nothing, ttm_sdpa_decode_static, through the C ABI against ttm_sdpa_decode_windowed (the
entry point it is a variant of): bit-identical output, two calls in a row on one GPU, the second with a smaller input, so
the second call finds the first call's partial results in the shared static array.  Sizes beyond the array are refused."""
import numpy as np
import pytest
import torch

from ttmlir_amd import datagen
from test_gpu_linear import tilize_dev, untilize_dev

pytestmark = pytest.mark.gpu


def _operands(hip, dev, B, H, Hkv, S, D, seed):
    q = datagen.randn((1, B, H, D), seed=seed, dtype=torch.bfloat16)
    k = datagen.randn((B, Hkv, S, D), seed=seed + 1, dtype=torch.bfloat16)
    v = datagen.randn((B, Hkv, S, D), seed=seed + 2, dtype=torch.bfloat16)
    return q, k, v, tilize_dev(hip, q, dev), tilize_dev(hip, k, dev), tilize_dev(hip, v, dev)


def _run(hip, name, qt, kt, vt, cp, B, H, Hkv, S, D, window=-1):
    out = torch.full_like(qt, float("nan"))
    hip.call(name, hip.ptr(qt), hip.ptr(kt), hip.ptr(vt), hip.ptr(cp), None, 1, 1, None, 0, 0, 0, hip.ptr(out), hip.BF16,
             B, H, Hkv, S, D, 1, 0.0, 0, window, None, hip.current_stream())
    torch.cuda.synchronize()
    return out


def test_static_scratch_decode_attention_equals_the_allocating_entry_point(hip, dev, orc):
    import oracle.metrics as metrics
    # first call: 8 users x 32 / 8 heads over 1024 positions; second call: smaller in every extent, and ragged positions
    for (B, H, Hkv, S, D, cur, window, seed) in [(8, 32, 8, 1024, 128, [1023, 5, 512, 700, 0, 31, 32, 999], -1, 70),
                                                  (3, 8, 2, 256, 64, [200, 0, 77], 64, 80)]:
        q, k, v, qt, kt, vt = _operands(hip, dev, B, H, Hkv, S, D, seed)
        cp = torch.tensor(cur, dtype=torch.int32, device=dev)
        got = _run(hip, "ttm_sdpa_decode_static", qt, kt, vt, cp, B, H, Hkv, S, D, window)
        ref = _run(hip, "ttm_sdpa_decode_windowed", qt, kt, vt, cp, B, H, Hkv, S, D, window)
        assert torch.equal(got.view(torch.int16), ref.view(torch.int16))      # same kernels, same bits
        assert bool(torch.isfinite(got.float()).all())
        want = orc.sdpa_decode(q.float().numpy(), k.float().numpy(), v.float().numpy(), cur_pos=cur, is_causal=True,
                               sliding_window=window if window >= 0 else None)
        have = untilize_dev(hip, got, q.shape, dev).float().cpu().numpy()
        assert np.max(np.abs(have - want)) <= 2.0 ** -6
        assert metrics.get_pcc(want, have) >= 0.9999


def test_static_scratch_refuses_what_does_not_fit(hip, dev):
    # 64 users x 32 kv heads x 8 heads per kv head over 8192 positions need more than the array's 8 MiB of partial results;
    # the check precedes every launch, so the small placeholder operands are never read
    z = torch.zeros(1024, dtype=torch.bfloat16, device=dev)
    cp = torch.zeros(64, dtype=torch.int32, device=dev)
    hip.set_option("check_extents", 0)     # the placeholders are far smaller than the operands the call names: that check would answer first
    try:
        with pytest.raises(hip.TTMError, match="static scratch holds"):
            hip.call("ttm_sdpa_decode_static", hip.ptr(z), hip.ptr(z), hip.ptr(z), hip.ptr(cp), None, 1, 1, None, 0, 0, 0, hip.ptr(z),
                     hip.BF16, 64, 256, 32, 8192, 128, 1, 0.0, 0, -1, None, hip.current_stream())
    finally:
        hip.set_option("check_extents", 1)
