"""Decode-path kernels through the C ABI against the CPU oracle: rotary embedding, KV-cache update / fill (bit exact:
they move or scale bf16 values the oracle reproduces exactly or within one rounding), attention of one token over a cache
(PCC >= 0.9999, max-abs stated)."""
import numpy as np
import pytest
import torch

from ttmlir_amd import datagen
from test_gpu_linear import tilize_dev, untilize_dev

pytestmark = pytest.mark.gpu


def f32(t):
    return t.float().cpu().numpy()


@pytest.mark.parametrize("B,H,S,D,cache_rows,token", [(1, 8, 64, 128, 64, None), (2, 4, 40, 64, 96, None), (1, 3, 7, 32, 32, None),
                                                       (1, 32, 32, 128, 2048, 1234), (4, 1, 8, 64, 64, 5)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rotary_embedding(hip, dev, orc, B, H, S, D, cache_rows, token, dtype):
    x = datagen.randn((B, H, S, D), seed=40, dtype=dtype)
    ang = datagen.randn((1, 1, cache_rows, D // 2), seed=41, dtype=torch.float32) * 2.0
    cos = torch.cat([ang.cos(), ang.cos()], -1).to(dtype)
    sin = torch.cat([ang.sin(), ang.sin()], -1).to(dtype)
    xt, ct, st = (tilize_dev(hip, t, dev) for t in (x, cos, sin))
    out = torch.full_like(xt, float("nan"))
    hip.call("ttm_rotary_embedding", hip.ptr(xt), hip.ptr(ct), hip.ptr(st), hip.ptr(out), hip.BF16 if dtype == torch.bfloat16 else hip.F32,
             B * H, S, D, cache_rows, -1 if token is None else token, hip.current_stream())
    got = f32(untilize_dev(hip, out, x.shape, dev))
    want = orc.rotary_embedding(f32(x), f32(cos), f32(sin), token_index=token)
    # two products and a sum, each rounded to fp32 (no fused multiply-add), as the CPU path's separate ops: bit exact
    assert np.array_equal(got, want if dtype == torch.float32 else orc.round_bf16(want))
    assert bool(torch.isfinite(out.float()).all())              # padding rows are written too (as zeros)


def test_rotary_embedding_rejects_bad_shapes(hip, dev):
    z = torch.zeros(32 * 48, dtype=torch.bfloat16, device=dev)
    with pytest.raises(hip.TTMError, match="multiple of 32"):
        hip.call("ttm_rotary_embedding", hip.ptr(z), hip.ptr(z), hip.ptr(z), hip.ptr(z), hip.BF16, 1, 32, 48, 32, -1, hip.current_stream())
    with pytest.raises(hip.TTMError, match="cached positions"):
        hip.call("ttm_rotary_embedding", hip.ptr(z), hip.ptr(z), hip.ptr(z), hip.ptr(z), hip.BF16, 1, 32, 32, 32, 32, hip.current_stream())
    with pytest.raises(hip.TTMError, match="caches hold"):
        hip.call("ttm_rotary_embedding", hip.ptr(z), hip.ptr(z), hip.ptr(z), hip.ptr(z), hip.BF16, 1, 33, 32, 32, -1, hip.current_stream())


@pytest.mark.parametrize("U,H,S,D,Bin,off,idx", [(1, 8, 128, 128, 1, 0, 5), (4, 2, 96, 64, 2, 1, 95), (32, 8, 64, 128, 32, 0, 33),
                                                  (2, 3, 40, 32, 1, 1, 39)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_update_cache_bit_exact(hip, dev, orc, U, H, S, D, Bin, off, idx, dtype):
    cache = datagen.randn((U, H, S, D), seed=42, dtype=dtype)
    upd = datagen.randn((1, H, Bin, D), seed=43, dtype=dtype)
    ct, ut = tilize_dev(hip, cache, dev), tilize_dev(hip, upd, dev)
    index = torch.tensor([idx], dtype=torch.int32, device=dev)
    code = hip.BF16 if dtype == torch.bfloat16 else hip.F32
    hip.call("ttm_update_cache", hip.ptr(ct), hip.ptr(ut), hip.ptr(index), code, U, H, S, D, Bin, off, hip.current_stream())
    got = f32(untilize_dev(hip, ct, cache.shape, dev))
    assert np.array_equal(got, orc.update_cache(f32(cache), f32(upd), idx, off))
    # an index outside the cache writes nothing
    before = ct.clone()
    index.fill_(S)
    hip.call("ttm_update_cache", hip.ptr(ct), hip.ptr(ut), hip.ptr(index), code, U, H, S, D, Bin, off, hip.current_stream())
    assert torch.equal(ct, before)
    with pytest.raises(hip.TTMError, match="outside the cache"):
        hip.call("ttm_update_cache", hip.ptr(ct), hip.ptr(ut), hip.ptr(index), code, U, H, S, D, Bin, U, hip.current_stream())


@pytest.mark.parametrize("U,H,S,D,seq,off", [(1, 8, 128, 128, 128, 0), (4, 2, 96, 64, 40, 3), (2, 3, 64, 32, 1, 1), (2, 1, 64, 64, 33, 0)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fill_cache_bit_exact(hip, dev, orc, U, H, S, D, seq, off, dtype):
    cache = datagen.randn((U, H, S, D), seed=44, dtype=dtype)
    fill = datagen.randn((1, H, seq, D), seed=45, dtype=dtype)
    ct, ft = tilize_dev(hip, cache, dev), tilize_dev(hip, fill, dev)
    hip.call("ttm_fill_cache", hip.ptr(ct), hip.ptr(ft), hip.BF16 if dtype == torch.bfloat16 else hip.F32, U, H, S, D, seq, off,
             hip.current_stream())
    got = f32(untilize_dev(hip, ct, cache.shape, dev))
    assert np.array_equal(got, orc.fill_cache(f32(cache), f32(fill), off))


def _decode_case(hip, dev, orc, B, H, Hkv, S, D, cur, mask_heads=None, causal=True, scale=0.0, paged=None, seed=50):
    import oracle.metrics as metrics
    q = datagen.randn((1, B, H, D), seed=seed, dtype=torch.bfloat16)
    k = datagen.randn((B, Hkv, S, D), seed=seed + 1, dtype=torch.bfloat16)
    v = datagen.randn((B, Hkv, S, D), seed=seed + 2, dtype=torch.bfloat16)
    m = datagen.randn((B, 1, mask_heads, S), seed=seed + 3, dtype=torch.bfloat16) if mask_heads else None
    cp = None if cur is None else torch.tensor(cur, dtype=torch.int32, device=dev)
    qt = tilize_dev(hip, q, dev)
    mt = tilize_dev(hip, m, dev) if m is not None else None
    table, pages, block = None, 0, 0
    if paged:
        # scatter the cache into shuffled pages [blocks, Hkv, block, D] behind a page table [B, S / block]
        block = paged
        pages = S // block
        perm = torch.randperm(B * pages, generator=torch.Generator().manual_seed(seed)).reshape(B, pages)
        kp = torch.zeros((B * pages, Hkv, block, D), dtype=torch.bfloat16)
        vp = torch.zeros_like(kp)
        for b in range(B):
            for j in range(pages):
                kp[perm[b, j]] = k[b, :, j * block:(j + 1) * block]
                vp[perm[b, j]] = v[b, :, j * block:(j + 1) * block]
        kt, vt = tilize_dev(hip, kp, dev), tilize_dev(hip, vp, dev)
        table = perm.to(torch.int32).to(dev)
    else:
        kt, vt = tilize_dev(hip, k, dev), tilize_dev(hip, v, dev)
    out = torch.full_like(qt, float("nan"))
    hip.call("ttm_sdpa_decode", hip.ptr(qt), hip.ptr(kt), hip.ptr(vt), hip.ptr(cp) if cp is not None else None,
             hip.ptr(mt) if mt is not None else None, mask_heads or 1, hip.ptr(table) if table is not None else None, pages, block, (B * pages if table is not None else 0),
             hip.ptr(out), hip.BF16, B, H, Hkv, S, D, int(causal), scale, hip.current_stream())
    got = f32(untilize_dev(hip, out, q.shape, dev))
    want = orc.sdpa_decode(f32(q), f32(k), f32(v), cur_pos=cur, mask=None if m is None else f32(m), is_causal=causal,
                           scale=scale or None)
    assert bool(torch.isfinite(out.float()).all())
    # fp32 scores and probabilities, output rounded to bf16 once: half a bf16 ulp of values up to ~4 plus summation order
    assert np.max(np.abs(got - want)) <= 2.0 ** -6, np.max(np.abs(got - want))
    assert metrics.get_pcc(want, got) >= 0.9999


@pytest.mark.parametrize("B,H,Hkv,S,D,cur", [
    (1, 32, 8, 2048, 128, [1500]),            # Llama-3-8B decode, one user
    (8, 32, 8, 1024, 128, [0, 1, 31, 32, 33, 500, 1022, 1023]),
    (32, 8, 8, 256, 64, list(range(0, 256, 8))),
    (2, 8, 1, 512, 32, [100, 511]),           # one kv head serving 8 query heads, single column tile
    (3, 12, 4, 96, 96, [95, 40, 7]),          # three column tiles
    (1, 16, 2, 8192, 256, [8000]),            # long cache: several slices per kv head
    (2, 32, 1, 512, 64, [300, 511]),          # multi-query attention: 32 query heads on one kv head, four launches of 8
    (3, 24, 2, 256, 128, [17, 200, 255]),     # 12 query heads per kv head: a launch of 8 and one of 4
])
def test_sdpa_decode_causal(hip, dev, orc, B, H, Hkv, S, D, cur):
    _decode_case(hip, dev, orc, B, H, Hkv, S, D, cur)


def test_sdpa_decode_mask_scale_and_full_attention(hip, dev, orc):
    _decode_case(hip, dev, orc, 2, 8, 2, 256, 64, None, causal=False)
    _decode_case(hip, dev, orc, 2, 8, 2, 256, 64, None, mask_heads=8, scale=0.2)
    _decode_case(hip, dev, orc, 2, 8, 2, 256, 64, None, mask_heads=1, scale=0.05)
    _decode_case(hip, dev, orc, 2, 8, 2, 256, 64, [7, 200], causal=False)       # positions are ignored without is_causal


@pytest.mark.parametrize("block", [32, 64, 256])
def test_sdpa_decode_paged(hip, dev, orc, block):
    _decode_case(hip, dev, orc, 4, 32, 8, 1024, 128, [3, 200, 640, 1023], paged=block)


def test_sdpa_decode_ignores_garbage_after_the_current_position(hip, dev, orc):
    # cache rows that were never written may hold NaN / Inf bit patterns: they must not leak into the output
    B, H, Hkv, S, D = 2, 8, 2, 512, 128
    q = datagen.randn((1, B, H, D), seed=60, dtype=torch.bfloat16)
    k = datagen.randn((B, Hkv, S, D), seed=61, dtype=torch.bfloat16)
    v = datagen.randn((B, Hkv, S, D), seed=62, dtype=torch.bfloat16)
    cur = [70, 300]
    kb, vb = k.clone(), v.clone()
    for b, c in enumerate(cur):
        kb[b, :, c + 1:] = float("nan")
        vb[b, :, c + 1:] = float("inf")
    cp = torch.tensor(cur, dtype=torch.int32, device=dev)
    qt, kt, vt = (tilize_dev(hip, t, dev) for t in (q, kb, vb))
    out = torch.full_like(qt, float("nan"))
    hip.call("ttm_sdpa_decode", hip.ptr(qt), hip.ptr(kt), hip.ptr(vt), hip.ptr(cp), None, 1, None, 0, 0, 0, hip.ptr(out), hip.BF16,
             B, H, Hkv, S, D, 1, 0.0, hip.current_stream())
    got = f32(untilize_dev(hip, out, q.shape, dev))
    want = orc.sdpa_decode(f32(q), f32(k), f32(v), cur_pos=cur)
    assert np.all(np.isfinite(got)) and np.max(np.abs(got - want)) <= 2.0 ** -6


def test_sdpa_decode_rejects_unsupported(hip, dev):
    z = torch.zeros(1 << 16, dtype=torch.bfloat16, device=dev)
    with pytest.raises(hip.TTMError, match="multiple of kv heads"):
        hip.call("ttm_sdpa_decode", hip.ptr(z), hip.ptr(z), hip.ptr(z), None, None, 1, None, 0, 0, 0, hip.ptr(z), hip.BF16, 1, 16, 3, 32, 32,
                 1, 0.0, hip.current_stream())
    with pytest.raises(hip.TTMError, match="multiple of 32"):
        hip.call("ttm_sdpa_decode", hip.ptr(z), hip.ptr(z), hip.ptr(z), None, None, 1, None, 0, 0, 0, hip.ptr(z), hip.BF16, 1, 8, 8, 40, 32,
                 1, 0.0, hip.current_stream())
    with pytest.raises(hip.TTMError, match="page table"):
        hip.call("ttm_sdpa_decode", hip.ptr(z), hip.ptr(z), hip.ptr(z), None, None, 1, hip.ptr(z), 3, 32, 8, hip.ptr(z), hip.BF16, 1, 8, 8,
                 64, 32, 1, 0.0, hip.current_stream())
    with pytest.raises(hip.TTMError, match="number of blocks"):
        hip.call("ttm_sdpa_decode", hip.ptr(z), hip.ptr(z), hip.ptr(z), None, None, 1, hip.ptr(z), 2, 32, 0, hip.ptr(z), hip.BF16, 1, 8, 8,
                 64, 32, 1, 0.0, hip.current_stream())


def test_sdpa_decode_page_table_entries_outside_the_cache_are_masked(hip, dev, orc):
    """Unused slots of a page table hold -1 (or stale numbers): a slot within [0, cur_pos] that names no block of the cache
    masks its keys instead of being followed, and slots past cur_pos are not looked at; non-causal calls mask them too."""
    B, H, Hkv, S, D, block = 3, 8, 2, 512, 64, 64
    pages = S // block
    q = datagen.randn((1, B, H, D), seed=150, dtype=torch.bfloat16)
    k = datagen.randn((B, Hkv, S, D), seed=151, dtype=torch.bfloat16)
    v = datagen.randn((B, Hkv, S, D), seed=152, dtype=torch.bfloat16)
    cur = [300, 511, 64]
    g = torch.Generator().manual_seed(153)
    table = torch.randperm(B * pages, generator=g).reshape(B, pages).to(torch.int32)
    kp = torch.zeros((B * pages, Hkv, block, D), dtype=torch.bfloat16)
    vp = torch.zeros_like(kp)
    for b in range(B):
        for pg in range(pages):
            kp[table[b, pg]] = k[b, :, pg * block:(pg + 1) * block]
            vp[table[b, pg]] = v[b, :, pg * block:(pg + 1) * block]
    bad = table.clone()
    bad[0, 5:] = -1                 # past user 0's position (300 is in page 4)
    bad[0, 2] = -1                  # inside it: keys 128..191 drop out
    bad[1, 7] = B * pages + 5       # beyond the cache: keys 448..511 drop out
    bad[2, 2:] = -1
    # what the kernel must do, written for the oracle as a mask (with a mask the golden leaves the position test to the
    # mask, tools/golden/mapping.py:2459-2470): keys past the position, and the keys of the two dropped pages
    mask = np.zeros((B, 1, 1, S), dtype=np.float32)
    for b in range(B):
        mask[b, ..., cur[b] + 1:] = -np.inf
    mask[0, ..., 128:192] = -np.inf
    mask[1, ..., 448:512] = -np.inf
    qt, kt, vt = tilize_dev(hip, q, dev), tilize_dev(hip, kp, dev), tilize_dev(hip, vp, dev)
    cp, td = torch.tensor(cur, dtype=torch.int32, device=dev), bad.to(dev)
    out = torch.full_like(qt, float("nan"))
    hip.call("ttm_sdpa_decode", hip.ptr(qt), hip.ptr(kt), hip.ptr(vt), hip.ptr(cp), None, 1, hip.ptr(td), pages, block, B * pages,
             hip.ptr(out), hip.BF16, B, H, Hkv, S, D, 1, 0.0, hip.current_stream())
    got = f32(untilize_dev(hip, out, q.shape, dev))
    want = orc.sdpa_decode(f32(q), f32(k), f32(v), cur_pos=cur, mask=mask, is_causal=True)
    assert np.all(np.isfinite(got)) and np.max(np.abs(got - want)) <= 2.0 ** -6
    plain = orc.sdpa_decode(f32(q), f32(k), f32(v), cur_pos=cur, is_causal=True)
    assert np.max(np.abs(plain[0, :2] - want[0, :2])) > 0.02       # the dropped pages matter


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("blocks,H,bs,D,users,pages,paged", [(12, 8, 64, 128, 4, 3, True), (40, 2, 32, 64, 32, 1, True), (6, 3, 96, 32, 5, 2, True),
                                                             (4, 8, 128, 128, 4, 0, False), (1, 2, 40, 64, 3, 0, False)])
def test_paged_update_cache_bit_exact(hip, dev, orc, dtype, blocks, H, bs, D, users, pages, paged):
    """ttm_paged_update_cache against the oracle: shuffled page tables, positions in every page, positions and block
    numbers out of range (nothing written), the static form with per-user entries and with one shared entry."""
    g = torch.Generator().manual_seed(60)
    cache = datagen.randn((blocks, H, bs, D), seed=61, dtype=dtype)
    inp = datagen.randn((1, users, H, D), seed=62, dtype=dtype)
    code = hip.BF16 if dtype == torch.bfloat16 else hip.F32
    cap = pages * bs if paged else bs
    pos = torch.randint(0, cap, (users,), generator=g, dtype=torch.int32)
    pos[0] = cap - 1
    if users > 2:
        pos[1], pos[2] = -1, cap                          # skipped users
    table = None
    if paged:
        table = torch.randperm(blocks, generator=g)[:users * pages].reshape(users, pages).to(torch.int32) if users * pages <= blocks \
            else torch.randint(0, blocks, (users, pages), generator=g, dtype=torch.int32)
        if users > 3:
            table[3, int(pos[3]) // bs] = blocks          # a block number past the cache
        # two users writing the same cell would race: keep (block, offset) unique among the writers
        seen = set()
        for u in range(users):
            if 0 <= int(pos[u]) < cap:
                key = (int(table[u, int(pos[u]) // bs]), int(pos[u]) % bs)
                if key in seen:
                    pos[u] = -1
                seen.add(key)
    shared = (not paged) and blocks == 1
    if shared:
        pos[:] = -1
        pos[users - 1] = 7                                # one writer into the shared entry
    ct, it = tilize_dev(hip, cache, dev), tilize_dev(hip, inp, dev)
    pos_d, table_d = pos.to(dev), table.to(dev) if paged else None       # kept alive across the launch
    hip.call("ttm_paged_update_cache", hip.ptr(ct), hip.ptr(it), hip.ptr(pos_d), hip.ptr(table_d) if paged else None, code,
             blocks, H, bs, D, users, pages, int(shared), hip.current_stream())
    got = f32(untilize_dev(hip, ct, cache.shape, dev))
    want = orc.paged_update_cache(f32(cache), f32(inp), pos.numpy(), table.numpy() if paged else None, share_cache=shared)
    assert np.array_equal(got, want)
    assert not np.array_equal(want, f32(cache))          # something was written


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("blocks,H,bs,D,batch,seq,rows,pages,with_idx", [(14, 8, 64, 128, 1, 200, 3, 4, True), (8, 2, 32, 64, 2, 64, 2, 2, False),
                                                                        (6, 3, 32, 32, 1, 33, 2, 1, True)])
def test_paged_fill_cache_bit_exact(hip, dev, orc, dtype, blocks, H, bs, D, batch, seq, rows, pages, with_idx):
    """ttm_paged_fill_cache against the oracle: a prefill longer than one block, ragged sequence lengths (the last block
    keeps its old rows past the sequence), sequences longer than the page table (the excess is dropped)."""
    g = torch.Generator().manual_seed(70)
    cache = datagen.randn((blocks, H, bs, D), seed=71, dtype=dtype)
    inp = datagen.randn((batch, H, seq, D), seed=72, dtype=dtype)
    code = hip.BF16 if dtype == torch.bfloat16 else hip.F32
    table = torch.randperm(blocks, generator=g)[:rows * pages].reshape(rows, pages).to(torch.int32)
    idx = torch.tensor([rows - 1] * batch, dtype=torch.int32) if with_idx else None
    ct, it = tilize_dev(hip, cache, dev), tilize_dev(hip, inp, dev)
    table_d, idx_d = table.to(dev), idx.to(dev) if with_idx else None    # kept alive across the launch
    hip.call("ttm_paged_fill_cache", hip.ptr(ct), hip.ptr(it), hip.ptr(table_d), hip.ptr(idx_d) if with_idx else None, code,
             blocks, H, bs, D, batch, seq, rows, pages, hip.current_stream())
    got = f32(untilize_dev(hip, ct, cache.shape, dev))
    want = orc.paged_fill_cache(f32(cache), f32(inp), table.numpy(), idx.numpy() if with_idx else None)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,H,D", [(32, 32, 128), (8, 8, 64), (5, 3, 32), (40, 2, 96)])
def test_rotary_embedding_split_heads_equals_reshape_then_rotary(hip, dev, dtype, B, H, D):
    """ttm_rotary_embedding_split_heads on the [users, heads * head_dim] matrix a projection leaves against the plain
    kernel on the reshaped tensor: bit-identical, padding rows zero."""
    x = datagen.randn((B, H * D), seed=80, dtype=dtype)
    cos = datagen.randn((1, 1, 4, D), seed=81, dtype=dtype)
    sin = datagen.randn((1, 1, 4, D), seed=82, dtype=dtype)
    code = hip.BF16 if dtype == torch.bfloat16 else hip.F32
    xt, ct, st = tilize_dev(hip, x, dev), tilize_dev(hip, cos, dev), tilize_dev(hip, sin, dev)
    x4 = tilize_dev(hip, x.reshape(1, B, H, D), dev)
    want = torch.full_like(x4, float("nan"))
    hip.call("ttm_rotary_embedding", hip.ptr(x4), hip.ptr(ct), hip.ptr(st), hip.ptr(want), code, B, H, D, 4, 2, hip.current_stream())
    got = torch.full_like(x4, float("nan"))
    hip.call("ttm_rotary_embedding_split_heads", hip.ptr(xt), hip.ptr(ct), hip.ptr(st), hip.ptr(got), code, B, H, D, 4, 2, hip.current_stream())
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    with pytest.raises(hip.TTMError, match="token_index"):
        hip.call("ttm_rotary_embedding_split_heads", hip.ptr(xt), hip.ptr(ct), hip.ptr(st), hip.ptr(got), code, B, H, D, 4, -1, hip.current_stream())


@pytest.mark.parametrize("B,H,Hkv,S,D", [(32, 32, 8, 512, 128), (5, 8, 2, 256, 64), (33, 4, 4, 128, 32), (4, 20, 1, 128, 32)])
def test_sdpa_decode_concat_heads_equals_reshape_of_the_plain_output(hip, dev, B, H, Hkv, S, D):
    """ttm_sdpa_decode_concat_heads writes [users, heads * head_dim]: the same values as ttm_sdpa_decode followed by a
    reshape, zero padding rows below the last user."""
    q = datagen.randn((1, B, H, D), seed=90, dtype=torch.bfloat16)
    k = datagen.randn((B, Hkv, S, D), seed=91, dtype=torch.bfloat16)
    v = datagen.randn((B, Hkv, S, D), seed=92, dtype=torch.bfloat16)
    cp = torch.randint(0, S, (B,), generator=torch.Generator().manual_seed(93), dtype=torch.int32).to(dev)
    qt, kt, vt = tilize_dev(hip, q, dev), tilize_dev(hip, k, dev), tilize_dev(hip, v, dev)
    plain = torch.full_like(qt, float("nan"))
    args = lambda out: (hip.ptr(qt), hip.ptr(kt), hip.ptr(vt), hip.ptr(cp), None, 1, None, 0, 0, 0, hip.ptr(out), hip.BF16, B, H, Hkv, S, D, 1, 0.0,
                        hip.current_stream())
    hip.call("ttm_sdpa_decode", *args(plain))
    Bp = (B + 31) // 32 * 32
    merged = torch.full((Bp * H * D,), float("nan"), dtype=torch.bfloat16, device=dev)
    hip.call("ttm_sdpa_decode_concat_heads", *args(merged))
    want = untilize_dev(hip, plain, q.shape, dev).reshape(B, H * D)
    got = untilize_dev(hip, merged, (B, H * D), dev)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert torch.equal(merged, tilize_dev(hip, want.cpu(), dev))          # padding rows are zero


@pytest.mark.parametrize("B,H,Hkv,S,D,window,sink,use_pos,paged,concat", [
    (4, 8, 2, 1024, 128, 128, False, True, False, 0), (4, 8, 2, 1024, 128, 1, False, True, False, 0),
    (3, 4, 4, 512, 64, 100, True, True, False, 0), (2, 8, 1, 2048, 128, 700, True, True, False, 1),
    (2, 4, 2, 256, 32, 40, True, False, False, 0), (5, 8, 2, 512, 128, 33, True, True, True, 0),
    (2, 20, 1, 256, 64, 64, True, True, False, 0), (32, 32, 8, 2048, 128, 512, False, True, False, 1),
    (2, 4, 2, 512, 128, None, True, True, False, 0), (2, 4, 2, 512, 128, 5000, False, True, False, 0),
    (1, 40, 40, 320, 96, 31, True, True, False, 0)])
def test_sdpa_decode_sliding_window_and_attention_sink(hip, dev, orc, B, H, Hkv, S, D, window, sink, use_pos, paged, concat):
    """ttm_sdpa_decode_windowed against the oracle: windows of one key, inside one slice of the cache, across slices,
    longer than the cache; with and without positions; the sink alone and with a window; paged caches, the merged output
    layout, more than 8 and more than 32 query heads.  The cache in front of every user's window holds NaN / Inf."""
    g = torch.Generator().manual_seed(130)
    q = datagen.randn((1, B, H, D), seed=131, dtype=torch.bfloat16)
    k = datagen.randn((B, Hkv, S, D), seed=132, dtype=torch.bfloat16)
    v = datagen.randn((B, Hkv, S, D), seed=133, dtype=torch.bfloat16)
    cur = torch.randint(0, S, (B,), generator=g, dtype=torch.int32)
    cur[0] = S - 1
    if B > 1:
        cur[1] = 0 if window is None else min(S - 1, max(0, window - 1))
    sk = (datagen.randn((H, 1), seed=134, dtype=torch.bfloat16) * 8).expand(H, 32).contiguous() if sink else None
    kb, vb = k.clone(), v.clone()
    for b in range(B):
        p = int(cur[b]) if use_pos else S - 1
        if use_pos:
            kb[b, :, p + 1:], vb[b, :, p + 1:] = float("nan"), float("inf")
        if window is not None and p - window + 1 > 0:
            kb[b, :, :p - window + 1], vb[b, :, :p - window + 1] = float("nan"), float("inf")
    table_d, pages, block = None, 0, 0
    if paged:
        block = 64
        pages = S // block
        table = torch.randperm(B * pages, generator=g).reshape(B, pages).to(torch.int32)
        kp = torch.empty((B * pages, Hkv, block, D), dtype=torch.bfloat16)
        vp = torch.empty_like(kp)
        for b in range(B):
            for pg in range(pages):
                kp[table[b, pg]] = kb[b, :, pg * block:(pg + 1) * block]
                vp[table[b, pg]] = vb[b, :, pg * block:(pg + 1) * block]
        kt, vt, table_d = tilize_dev(hip, kp, dev), tilize_dev(hip, vp, dev), table.to(dev)
    else:
        kt, vt = tilize_dev(hip, kb, dev), tilize_dev(hip, vb, dev)
    qt = tilize_dev(hip, q, dev)
    st = tilize_dev(hip, sk, dev) if sink else None
    cp = cur.to(dev)
    Bp = (B + 31) // 32 * 32
    out = torch.full((Bp * H * D,), float("nan"), dtype=torch.bfloat16, device=dev) if concat else torch.full_like(qt, float("nan"))
    hip.call("ttm_sdpa_decode_windowed", hip.ptr(qt), hip.ptr(kt), hip.ptr(vt), hip.ptr(cp) if use_pos else None, None, 1, 1,
             hip.ptr(table_d) if paged else None, pages, block, B * pages, hip.ptr(out), hip.BF16, B, H, Hkv, S, D, 1, 0.0, concat,
             -1 if window is None else window, hip.ptr(st) if sink else None, hip.current_stream())
    got = f32(untilize_dev(hip, out, (B, H * D), dev)).reshape(1, B, H, D) if concat else f32(untilize_dev(hip, out, q.shape, dev))
    want = orc.sdpa_decode(f32(q), f32(k), f32(v), cur_pos=cur.numpy() if use_pos else None, sliding_window=window,
                           attention_sink=None if sk is None else f32(sk))
    assert np.all(np.isfinite(got)) and np.max(np.abs(got - want)) <= 2.0 ** -6
    if window is not None and window < S // 2 and not sink:
        plain = orc.sdpa_decode(f32(q), f32(k), f32(v), cur_pos=cur.numpy() if use_pos else None)
        assert np.max(np.abs(plain - want)) > 0.02           # the window matters for this case


@pytest.mark.parametrize("mask_batch,mask_heads", [(1, 1), (1, 8), (3, 1), (3, 8)])
def test_sdpa_decode_mask_shared_by_the_users(hip, dev, orc, mask_batch, mask_heads):
    """The decode op's mask is [1|batch, 1, 1|heads, positions] (include/ttmlir/Dialect/TTNN/IR/TTNNOps.td:4123-4125):
    every combination of shared and per-user, shared and per-head, with a window and a sink on top, against the oracle
    on the broadcast mask."""
    B, H, Hkv, S, D = 3, 8, 2, 256, 64
    q = datagen.randn((1, B, H, D), seed=140, dtype=torch.bfloat16)
    k = datagen.randn((B, Hkv, S, D), seed=141, dtype=torch.bfloat16)
    v = datagen.randn((B, Hkv, S, D), seed=142, dtype=torch.bfloat16)
    m = datagen.randn((mask_batch, 1, mask_heads, S), seed=143, dtype=torch.bfloat16) * 4
    m[..., 200:] = float("-inf")
    sk = (datagen.randn((H, 1), seed=144, dtype=torch.bfloat16) * 4).expand(H, 32).contiguous()
    qt, kt, vt, mt, st = (tilize_dev(hip, t, dev) for t in (q, k, v, m, sk))
    out = torch.full_like(qt, float("nan"))
    hip.call("ttm_sdpa_decode_windowed", hip.ptr(qt), hip.ptr(kt), hip.ptr(vt), None, hip.ptr(mt), mask_heads, mask_batch, None, 0, 0, 0,
             hip.ptr(out), hip.BF16, B, H, Hkv, S, D, 0, 0.0, 0, 100, hip.ptr(st), hip.current_stream())
    got = f32(untilize_dev(hip, out, q.shape, dev))
    want = orc.sdpa_decode(f32(q), f32(k), f32(v), mask=f32(m), is_causal=False, sliding_window=100, attention_sink=f32(sk))
    assert np.all(np.isfinite(got)) and np.max(np.abs(got - want)) <= 2.0 ** -6


@pytest.mark.parametrize("users,K,H,Hkv,D,S,pos,off,cache_users,token,rows", [
    (32, 4096, 32, 8, 128, 2048, 2047, 0, 32, 0, 1),      # the Llama-3-8B decode step
    (5, 256, 4, 2, 64, 96, 33, 1, 8, 2, 4),               # ragged users, padded heads, batch offset, a row of a longer cos cache
    (1, 512, 8, 8, 32, 32, 0, 0, 1, 0, 1),
    (32, 1024, 8, 1, 128, 64, 70, 0, 32, 0, 1),           # position outside the cache: q comes out, the caches stay
])
@pytest.mark.parametrize("fmt", ["bfp8", "bfp4"])
def test_linear_qkv_decode_equals_the_op_sequence(hip, dev, orc, users, K, H, Hkv, D, S, pos, off, cache_users, token, rows, fmt):
    """ttm_linear_qkv_decode against the ops it stands for, run one by one through the C ABI (ttm_linear_group, two
    ttm_rotary_embedding_split_heads, the cache rows written by hand): bit-identical q and caches; and q against the oracle."""
    from test_gpu_linear import pack_weight
    wf = hip.BFP8B if fmt == "bfp8" else hip.BFP4B
    a = datagen.randn((users, K), seed=90, dtype=torch.bfloat16)
    ws = [datagen.randn((K, n * D), seed=91 + i, dtype=torch.float32) * 0.05 for i, n in enumerate((H, Hkv, Hkv))]
    ang = datagen.randn((1, 1, rows, D // 2), seed=95, dtype=torch.float32) * 2.0
    cos = torch.cat([ang.cos(), ang.cos()], -1).to(torch.bfloat16)
    sin = torch.cat([ang.sin(), ang.sin()], -1).to(torch.bfloat16)
    caches = [datagen.randn((cache_users, Hkv, S, D), seed=96 + i, dtype=torch.bfloat16) for i in range(2)]
    at, ct, st = tilize_dev(hip, a, dev), tilize_dev(hip, cos, dev), tilize_dev(hip, sin, dev)
    wt = [pack_weight(hip, w, wf, dev) for w in ws]
    index = torch.tensor([pos], dtype=torch.int32, device=dev)
    s = hip.current_stream()
    # the op sequence; the three projections share a launch as they do in a program (a projection launched alone may split
    # K another way and round a few sums to the neighbouring bf16 value)
    import ctypes
    lin = [torch.full((32 * n * D,), float("nan"), dtype=torch.bfloat16, device=dev) for n in (H, Hkv, Hkv)]
    wp = (ctypes.c_void_p * 3)(*[t.data_ptr() for t in wt])
    op = (ctypes.c_void_p * 3)(*[t.data_ptr() for t in lin])
    nn = (ctypes.c_int64 * 3)(H * D, Hkv * D, Hkv * D)
    hip.call("ttm_linear_group", hip.ptr(at), 3, wp, wf, op, nn, None, users, K, s)
    rot = []
    for o, n in zip(lin[:2], (H, Hkv)):
        r = torch.full((users * ((n + 31) // 32 * 32) * D,), float("nan"), dtype=torch.bfloat16, device=dev)
        hip.call("ttm_rotary_embedding_split_heads", hip.ptr(o), hip.ptr(ct), hip.ptr(st), hip.ptr(r), hip.BF16, users, n, D, rows, token, s)
        rot.append(r)
    k_rot = untilize_dev(hip, rot[1], (1, users, Hkv, D), dev)
    v_lin = untilize_dev(hip, lin[2], (users, Hkv * D), dev).reshape(1, users, Hkv, D)
    want_caches = [c.clone().to(dev) for c in caches]
    if 0 <= pos < S:
        want_caches[0][off:off + users, :, pos, :] = k_rot[0]
        want_caches[1][off:off + users, :, pos, :] = v_lin[0]
    # the fused entry point
    assert hip.lib().ttm_linear_qkv_decode_supported(wf, users, K, H, Hkv, D) == 1
    q = torch.full_like(rot[0], float("nan"))
    ck, cv = (tilize_dev(hip, c, dev) for c in caches)
    hip.call("ttm_linear_qkv_decode", hip.ptr(at), hip.ptr(wt[0]), hip.ptr(wt[1]), hip.ptr(wt[2]), wf, users, K, H, Hkv, D, hip.ptr(ct),
             hip.ptr(st), rows, token, hip.ptr(q), hip.ptr(ck), hip.ptr(cv), cache_users, S, hip.ptr(index), off, s)
    torch.cuda.synchronize()
    assert torch.equal(q, rot[0])                                       # padding rows of q included (zeros)
    assert torch.equal(untilize_dev(hip, ck, caches[0].shape, dev), want_caches[0])
    assert torch.equal(untilize_dev(hip, cv, caches[1].shape, dev), want_caches[1])
    # q against the oracle: projection on the dequantised weights, bf16, rotary embedding, bf16
    back = torch.empty(ws[0].shape, dtype=torch.float32, device=dev)
    hip.call("ttm_bfp_unpack", hip.ptr(wt[0]), wf, hip.ptr(back), hip.F32, hip.ROW_MAJOR, 1, K, H * D, s)
    proj = orc.round_bf16(orc.linear(f32(a), f32(back)))
    want_q = orc.round_bf16(orc.rotary_embedding(proj.reshape(1, users, H, D), f32(cos), f32(sin), token_index=token))
    got_q = f32(untilize_dev(hip, q, (1, users, H, D), dev))
    # the projection differs from the oracle's at bf16 ties of its fp32 sums (another summation order); where it agrees the
    # rotary embedding is the oracle's arithmetic exactly
    assert np.mean(got_q == want_q) > 0.98
    assert np.max(np.abs(got_q - want_q)) <= 2.0 ** -7 * max(1.0, float(np.max(np.abs(want_q))))


def test_linear_qkv_decode_rejects_what_it_cannot_fuse(hip, dev):
    z = torch.zeros(32 * 64, dtype=torch.bfloat16, device=dev)
    args = lambda users=4, D=64, token=0, rows=1, off=0, cu=4: (hip.ptr(z), hip.ptr(z), hip.ptr(z), hip.ptr(z), hip.BFP8B, users, 64, 1, 1, D,
                                                                 hip.ptr(z), hip.ptr(z), rows, token, hip.ptr(z), hip.ptr(z), hip.ptr(z), cu, 32,
                                                                 hip.ptr(z), off, hip.current_stream())
    assert hip.lib().ttm_linear_qkv_decode_supported(hip.BFP8B, 33, 64, 1, 1, 64) == 0
    assert hip.lib().ttm_linear_qkv_decode_supported(hip.BF16, 4, 64, 1, 1, 64) == 0
    assert hip.lib().ttm_linear_qkv_decode_supported(hip.BFP8B, 4, 64, 1, 1, 48) == 0
    with pytest.raises(hip.TTMError, match="1..32 users"):
        hip.call("ttm_linear_qkv_decode", *args(users=33))
    with pytest.raises(hip.TTMError, match="token_index"):
        hip.call("ttm_linear_qkv_decode", *args(token=1))
    with pytest.raises(hip.TTMError, match="exceeds the cache"):
        hip.call("ttm_linear_qkv_decode", *args(off=1))


@pytest.mark.parametrize("M,K,N,fmt,with_w,with_b", [
    (32, 4096, 4096, "bfp8", True, False),      # the output projection of the Llama-3-8B decode step (K split four ways)
    (7, 256, 512, "bfp8", True, True),          # no split, ragged rows
    (32, 14336, 4096, "bfp4", True, False),
    (1, 512, 96, "bfp4", False, False),
])
def test_linear_add_rms_norm_equals_the_op_sequence(hip, dev, orc, M, K, N, fmt, with_w, with_b):
    """ttm_linear_add_rms_norm against ttm_linear_tail (add) followed by ttm_rms_norm: both outputs bit-identical."""
    from test_gpu_linear import pack_weight
    wf = hip.BFP8B if fmt == "bfp8" else hip.BFP4B
    a = datagen.randn((M, K), seed=110, dtype=torch.bfloat16)
    w = datagen.randn((K, N), seed=111, dtype=torch.float32) * 0.05
    res = datagen.randn((M, N), seed=112, dtype=torch.bfloat16)
    nw = (1.0 + 0.1 * datagen.randn((1, N), seed=113, dtype=torch.float32)).to(torch.bfloat16)
    nb = (0.1 * datagen.randn((1, N), seed=114, dtype=torch.float32)).to(torch.bfloat16)
    at, rt_, wt, nwt, nbt = tilize_dev(hip, a, dev), tilize_dev(hip, res, dev), pack_weight(hip, w, wf, dev), tilize_dev(hip, nw, dev), tilize_dev(hip, nb, dev)
    s = hip.current_stream()
    Np = (N + 31) // 32 * 32
    x1 = torch.full((32 * Np,), float("nan"), dtype=torch.bfloat16, device=dev)
    h = torch.full_like(x1, float("nan"))
    hip.call("ttm_linear_tail", hip.ptr(at), hip.BF16, hip.ptr(wt), wf, 0, None, hip.BF16, hip.TILE, hip.ptr(x1), hip.BF16, 1, 1, M, N, K,
             hip.ACT[None], 1, hip.ptr(rt_), s)
    hip.call("ttm_rms_norm", hip.ptr(x1), hip.ptr(nwt) if with_w else None, hip.TILE, hip.ptr(nbt) if with_b else None, hip.TILE, hip.ptr(h),
             hip.BF16, 1, M, N, 1e-5, s)
    assert hip.lib().ttm_linear_add_rms_norm_supported(wf, M, N, K) == 1
    x1f, hf = torch.full_like(x1, float("nan")), torch.full_like(x1, float("nan"))
    hip.call("ttm_linear_add_rms_norm", hip.ptr(at), hip.ptr(wt), wf, hip.ptr(rt_), hip.ptr(x1f), hip.ptr(nwt) if with_w else None, hip.TILE,
             hip.ptr(nbt) if with_b else None, hip.TILE, 1e-5, hip.ptr(hf), M, N, K, s)
    torch.cuda.synchronize()
    assert torch.equal(x1f, x1) and torch.equal(hf, h)
    assert bool(torch.isfinite(hf.float()).all())
    assert hip.lib().ttm_linear_add_rms_norm_supported(wf, 33, N, K) == 0 and hip.lib().ttm_linear_add_rms_norm_supported(hip.BF16, M, N, K) == 0
    with pytest.raises(hip.TTMError, match="must not alias"):
        hip.call("ttm_linear_add_rms_norm", hip.ptr(at), hip.ptr(wt), wf, hip.ptr(rt_), hip.ptr(rt_), None, hip.TILE, None, hip.TILE, 1e-5,
                 hip.ptr(hf), M, N, K, s)


@pytest.mark.parametrize("M,K,N,fmt,acts", [
    (32, 4096, 14336, "bfp8", ("silu", None)),     # gate and up of the Llama-3-8B decode step
    (32, 4096, 14336, "bfp4", ("silu", None)),
    (7, 256, 1000, "bfp8", ("gelu", "relu")),      # ragged rows and columns, an odd number of column tiles
    (1, 512, 96, "bfp4", (None, "sigmoid")),
    (32, 1024, 8224, "bfp8", ("silu", None)),      # 129 column pairs: the first width at which K = 1024 is not split
])
def test_linear_glu_equals_the_op_sequence(hip, dev, orc, M, K, N, fmt, acts):
    """ttm_linear_glu against ttm_linear (gate) followed by ttm_linear_tail (up, multiply): bit-identical, padding rows of the
    output left alone; and against the CPU oracle's linear + multiply with the three bf16 roundings."""
    from test_gpu_linear import pack_weight
    wf = hip.BFP8B if fmt == "bfp8" else hip.BFP4B
    a = datagen.randn((M, K), seed=120, dtype=torch.bfloat16)
    wg = datagen.randn((K, N), seed=121, dtype=torch.float32) * 0.05
    wu = datagen.randn((K, N), seed=122, dtype=torch.float32) * 0.05
    at, wgt, wut = tilize_dev(hip, a, dev), pack_weight(hip, wg, wf, dev), pack_weight(hip, wu, wf, dev)
    s = hip.current_stream()
    Np = (N + 31) // 32 * 32
    gate = torch.zeros((32 * Np,), dtype=torch.bfloat16, device=dev)
    want = torch.zeros_like(gate)
    hip.call("ttm_linear", hip.ptr(at), hip.BF16, hip.ptr(wgt), wf, 0, None, hip.BF16, hip.TILE, hip.ptr(gate), hip.BF16, 1, 1, M, N, K,
             hip.ACT[acts[0]], s)
    hip.call("ttm_linear_tail", hip.ptr(at), hip.BF16, hip.ptr(wut), wf, 0, None, hip.BF16, hip.TILE, hip.ptr(want), hip.BF16, 1, 1, M, N, K,
             hip.ACT[acts[1]], 2, hip.ptr(gate), s)
    assert hip.lib().ttm_linear_glu_supported(wf, M, N, K) == 1
    got = torch.zeros_like(want)
    hip.call("ttm_linear_glu", hip.ptr(at), hip.ptr(wgt), hip.ptr(wut), wf, hip.ptr(got), M, N, K, hip.ACT[acts[0]], hip.ACT[acts[1]], s)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert bool(torch.isfinite(got.float()).all())
    # the oracle on the weights the device multiplies
    r = lambda x: orc.round_bf16(x)
    fmtn = 8 if fmt == "bfp8" else 4
    q = lambda w_: orc.bfp_unpack(orc.bfp_pack(w_.numpy(), fmtn), w_.shape, fmtn)
    an = a.float().numpy()
    ref = r(r(orc.linear(an, q(wg), None, acts[0])) * r(orc.linear(an, q(wu), None, acts[1])))
    out = untilize_dev(hip, got, (32, Np), dev)[:M, :N].float().cpu().numpy()
    assert np.max(np.abs(out - ref)) <= 2.0 ** -5 * max(1.0, float(np.max(np.abs(ref))))
    assert hip.lib().ttm_linear_glu_supported(wf, 33, N, K) == 0 and hip.lib().ttm_linear_glu_supported(hip.BF16, M, N, K) == 0
    # a width at which one projection alone splits K over workgroups stays with the op sequence
    assert hip.lib().ttm_linear_glu_supported(wf, 32, 4096, 4096) == 0
    with pytest.raises(hip.TTMError, match="ttm_linear_glu"):
        hip.call("ttm_linear_glu", hip.ptr(at), hip.ptr(wgt), hip.ptr(wut), wf, hip.ptr(got), 33, N, K, 0, 0, s)


@pytest.mark.parametrize("M,K,N,acts", [
    (512, 4096, 14336, ("silu", None)),      # gate and up of config 4
    (100, 256, 1000, ("gelu", "relu")),       # ragged rows and columns: 32 column tiles = four blocks of eight tile slots
    (1024, 512, 544, (None, "sigmoid")),      # 17 column tiles: the last block holds one tile of either matrix
    (65, 96, 96, ("silu", None)),             # the smallest row count of the form, a ragged k tile pair
])
def test_linear_glu_main_kernel_equals_the_op_sequence(hip, dev, orc, M, K, N, acts):
    """ttm_linear_glu at 65..1024 rows (the fused main kernel over alternating column tiles of the two bfp8_b matrices, the
    product taken in the epilogue) against ttm_linear (gate) + ttm_linear_tail (up, multiply) on the same kernel without
    split K: bit-identical; and against the CPU oracle with the three bf16 roundings."""
    from test_gpu_linear import pack_weight
    wf = hip.BFP8B
    a = datagen.randn((M, K), seed=140, dtype=torch.bfloat16)
    wg = datagen.randn((K, N), seed=141, dtype=torch.float32) * 0.05
    wu = datagen.randn((K, N), seed=142, dtype=torch.float32) * 0.05
    at, wgt, wut = tilize_dev(hip, a, dev), pack_weight(hip, wg, wf, dev), pack_weight(hip, wu, wf, dev)
    s = hip.current_stream()
    Mp, Np = (M + 31) // 32 * 32, (N + 31) // 32 * 32
    gate = torch.zeros((Mp * Np,), dtype=torch.bfloat16, device=dev)
    want = torch.zeros_like(gate)
    got = torch.zeros_like(want)
    try:   # one pass and no split K for the op sequence; with the image pass ruled out the gated form takes every shape it can run
        hip.set_option("linear_split_k", 1)
        hip.set_option("linear_two_pass", 1)
        hip.call("ttm_linear", hip.ptr(at), hip.BF16, hip.ptr(wgt), wf, 0, None, hip.BF16, hip.TILE, hip.ptr(gate), hip.BF16, 1, 1, M, N, K,
                 hip.ACT[acts[0]], s)
        hip.call("ttm_linear_tail", hip.ptr(at), hip.BF16, hip.ptr(wut), wf, 0, None, hip.BF16, hip.TILE, hip.ptr(want), hip.BF16, 1, 1, M, N, K,
                 hip.ACT[acts[1]], 2, hip.ptr(gate), s)
        assert hip.lib().ttm_linear_glu_supported(wf, M, N, K) == 1
        hip.call("ttm_linear_glu", hip.ptr(at), hip.ptr(wgt), hip.ptr(wut), wf, hip.ptr(got), M, N, K, hip.ACT[acts[0]], hip.ACT[acts[1]], s)
        torch.cuda.synchronize()
    finally:
        hip.set_option("linear_split_k", 0)
        hip.set_option("linear_two_pass", 0)
    g2, w2 = untilize_dev(hip, got, (Mp, Np), dev)[:M, :N], untilize_dev(hip, want, (Mp, Np), dev)[:M, :N]
    assert torch.equal(g2, w2)
    assert bool(torch.isfinite(g2.float()).all())
    r = lambda x: orc.round_bf16(x)
    q = lambda w_: orc.bfp_unpack(orc.bfp_pack(w_.numpy(), 8), w_.shape, 8)
    an = a.float().numpy()
    orc.set_threads(orc.max_threads())
    try:
        ref = r(r(orc.linear(an, q(wg), None, acts[0])) * r(orc.linear(an, q(wu), None, acts[1])))
    finally:
        orc.set_threads(1)
    out = g2.float().cpu().numpy()
    assert np.max(np.abs(out - ref)) <= 2.0 ** -5 * max(1.0, float(np.max(np.abs(ref))))
    # bfp4_b weights and the token counts between the two forms stay with the op sequence
    assert hip.lib().ttm_linear_glu_supported(hip.BFP4B, M, N, K) == 0 and hip.lib().ttm_linear_glu_supported(wf, 48, N, K) == 0
    assert hip.lib().ttm_linear_glu_supported(wf, 2048, N, K) == 0
    # by default it weighs the library's model of the image pass against the multiply it saves: config 4's shape takes the gated
    # kernel up to 1024 rows, a square weight (cheap to rewrite as images, few blocks for the gated kernel) does not
    assert hip.lib().ttm_linear_glu_supported(wf, 512, 14336, 4096) == 1 and hip.lib().ttm_linear_glu_supported(wf, 1024, 14336, 4096) == 1
    assert hip.lib().ttm_linear_glu_supported(wf, 512, 4096, 4096) == 0
