"""GPU parity: tilize / untilize and bfp8_b / bfp4_b pack / unpack through the C ABI, bit exact
against the CPU oracle on the same seeded inputs, plus size-independent properties at the
full benchmark size (8192 x 8192)."""
import numpy as np
import pytest
import torch

from ttmlir_amd import datagen

pytestmark = pytest.mark.gpu

NP2T = {np.dtype(np.float32): torch.float32, np.dtype(np.uint16): torch.int16, np.dtype(np.uint8): torch.uint8,
        np.dtype(np.int32): torch.int32}


def to_dev(x, dev):
    return torch.from_numpy(x.view(np.int16) if x.dtype == np.uint16 else x).to(dev)


def run_tilize(hip, dev, x, variant=0, untilize_shape=None):
    b, r, c = x.shape[:-2], x.shape[-2], x.shape[-1]
    batch = int(np.prod(b, dtype=np.int64))
    pr, pc = (r + 31) // 32 * 32, (c + 31) // 32 * 32
    xd = to_dev(x, dev)
    out = torch.full((batch * pr * pc,), 0x55, dtype=xd.dtype, device=dev)
    hip.set_option("tilize_variant", variant)
    hip.call("ttm_tilize", hip.ptr(xd), hip.ptr(out), batch, r, c, x.dtype.itemsize, hip.current_stream())
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("variant", [0, 1])
@pytest.mark.parametrize("shape,dtype", [((256, 512), np.uint16), ((512, 256), np.uint16), ((64, 128), np.float32),
                                         ((3, 64, 256), np.float32), ((2, 2, 32, 32), np.uint8),
                                         ((96, 1536), np.uint8), ((1024, 1024), np.float32)])
def test_tilize_untilize_bit_exact(hip, dev, orc, shape, dtype, variant):
    rng = np.random.default_rng(0)
    x = rng.integers(0, 2 ** (8 * np.dtype(dtype).itemsize) - 1, size=shape, dtype=np.uint64).astype(
        np.uint32).astype(dtype) if dtype != np.float32 else rng.standard_normal(shape).astype(np.float32)
    t = run_tilize(hip, dev, x, variant)
    want = orc.tilize(x)
    got = t.cpu().numpy().view(x.dtype)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    # and back
    back = torch.empty_like(to_dev(x, dev))
    hip.set_option("untilize_variant", variant)
    batch = int(np.prod(shape[:-2], dtype=np.int64))
    hip.call("ttm_untilize", hip.ptr(t), hip.ptr(back), batch, shape[-2], shape[-1], x.dtype.itemsize,
             hip.current_stream())
    torch.cuda.synchronize()
    assert np.array_equal(back.cpu().numpy().view(x.dtype).view(np.uint8), x.view(np.uint8))


@pytest.mark.parametrize("dtype", [np.float32, np.uint16, np.uint8])
@pytest.mark.parametrize("shape", [(1, 1), (5, 7), (33, 31), (3, 17, 40), (1, 100), (40, 4096), (3, 500, 1000), (2, 70, 1002), (65, 33),
                                   (2, 2, 31, 64)])
def test_tilize_ragged_zero_padded(hip, dev, orc, shape, dtype):
    """Shapes that are not multiples of 32 in 4-, 2- and 1-byte elements: rows whose row-major start is 16-byte aligned in
    every row, in every other row, in none; batches; the padding of the tiles is zero, untilize leaves nothing outside the
    row-major tensor (the buffer is longer than it and must keep its fill)."""
    rng = np.random.default_rng(1)
    x = rng.standard_normal(shape).astype(np.float32) if dtype == np.float32 else rng.integers(1, 250, shape).astype(dtype)
    t = run_tilize(hip, dev, x)
    assert np.array_equal(t.cpu().numpy().view(dtype), orc.tilize(x).view(dtype).reshape(-1))
    n = int(np.prod(shape))
    back = torch.full((n + 64,), 7, dtype=t.dtype, device=dev)
    b, r, c = orc._split3(shape)
    hip.call("ttm_untilize", hip.ptr(t), hip.ptr(back), b, r, c, x.dtype.itemsize, hip.current_stream())
    torch.cuda.synchronize()
    got = back.cpu().numpy().view(dtype)
    assert np.array_equal(got[:n].reshape(shape), x)
    assert np.all(got[n:] == np.asarray(7, dtype=back.cpu().numpy().dtype).view(dtype))


def test_c1_operands_layout(hip, dev, orc):
    a, b = datagen.c1_matmul()
    for m in (a, b):
        x = m.view(torch.int16).numpy().view(np.uint16)
        t = run_tilize(hip, dev, x)
        assert np.array_equal(t.cpu().numpy().view(np.uint16), orc.tilize(x))


def pack_gpu(hip, dev, xd, fmt, shape, dtype, layout):
    b, r, c = shape
    pr, pc = (r + 31) // 32 * 32, (c + 31) // 32 * 32
    nt = b * (pr // 32) * (pc // 32)
    out = torch.full((nt * hip.bfp_tile_bytes(fmt),), 0x55, dtype=torch.uint8, device=dev)
    hip.call("ttm_bfp_pack", hip.ptr(xd), dtype, layout, hip.ptr(out), fmt, b, r, c, hip.current_stream())
    return out


def unpack_gpu(hip, dev, pd, fmt, shape, dtype, layout):
    b, r, c = shape
    pr, pc = (r + 31) // 32 * 32, (c + 31) // 32 * 32
    n = b * r * c if layout == hip.ROW_MAJOR else b * pr * pc
    out = torch.full((n,), -7, dtype=torch.float32 if dtype == hip.F32 else torch.bfloat16, device=dev)
    hip.call("ttm_bfp_unpack", hip.ptr(pd), fmt, hip.ptr(out), dtype, layout, b, r, c, hip.current_stream())
    return out


@pytest.mark.parametrize("fmt", [8, 4])
@pytest.mark.parametrize("shape", [(1, 32, 32), (1, 256, 512), (2, 64, 96), (1, 40, 50), (3, 1, 33), (1, 1024, 1024)])
def test_bfp_pack_unpack_f32_rowmajor(hip, dev, orc, fmt, shape):
    hfmt = hip.BFP8B if fmt == 8 else hip.BFP4B
    x = datagen.c2_outliers(shape[0] * shape[1], shape[2], seed=3).reshape(shape)
    x[0, 0, : min(4, shape[2])] = 0.0
    xd = x.to(dev)
    pd = pack_gpu(hip, dev, xd, hfmt, shape, hip.F32, hip.ROW_MAJOR)
    want = orc.bfp_pack(x.numpy(), fmt)
    torch.cuda.synchronize()
    assert np.array_equal(pd.cpu().numpy(), want)
    back = unpack_gpu(hip, dev, pd, hfmt, shape, hip.F32, hip.ROW_MAJOR)
    torch.cuda.synchronize()
    want_back = orc.bfp_unpack(want, shape, fmt)
    assert np.array_equal(back.cpu().numpy().view(np.uint32), want_back.reshape(-1).view(np.uint32))


@pytest.mark.parametrize("fmt", [8, 4])
def test_bfp_tiled_and_bf16_sides(hip, dev, orc, fmt):
    hfmt = hip.BFP8B if fmt == 8 else hip.BFP4B
    shape = (2, 64, 128)
    x = datagen.c2_outliers(128, 128, seed=5).reshape(shape)
    xb = x.to(torch.bfloat16)
    want = orc.bfp_pack(xb.float().numpy(), fmt)          # bf16 sources are widened exactly
    # bf16 row-major source
    pd = pack_gpu(hip, dev, xb.to(dev), hfmt, shape, hip.BF16, hip.ROW_MAJOR)
    torch.cuda.synchronize()
    assert np.array_equal(pd.cpu().numpy(), want)
    # fp32 tile-ordered source
    tiled = torch.from_numpy(orc.tilize(xb.float().numpy())).to(dev)
    pd2 = pack_gpu(hip, dev, tiled, hfmt, shape, hip.F32, hip.TILE)
    # bf16 tile-ordered source
    pd3 = pack_gpu(hip, dev, tiled.to(torch.bfloat16), hfmt, shape, hip.BF16, hip.TILE)
    torch.cuda.synchronize()
    assert np.array_equal(pd2.cpu().numpy(), want) and np.array_equal(pd3.cpu().numpy(), want)
    # unpack to every plain side
    vals = orc.bfp_unpack(want, shape, fmt)
    u1 = unpack_gpu(hip, dev, pd, hfmt, shape, hip.BF16, hip.ROW_MAJOR)
    u2 = unpack_gpu(hip, dev, pd, hfmt, shape, hip.F32, hip.TILE)
    u3 = unpack_gpu(hip, dev, pd, hfmt, shape, hip.BF16, hip.TILE)
    torch.cuda.synchronize()
    assert np.array_equal(u1.float().cpu().numpy(), vals.reshape(-1))      # bf16 holds decoded values exactly
    assert np.array_equal(u2.cpu().numpy(), orc.tilize(vals))
    assert np.array_equal(u3.float().cpu().numpy(), orc.tilize(vals))


def test_bfp_special_values(hip, dev, orc):
    x = np.zeros((32, 32), dtype=np.float32)
    x[0, :8] = [1.0, 0.5, -0.25, 1.9921875, 1.984375, 0.0078125, -0.00390625, 0.01171875]
    x[1, :4] = [1e-40, -1e-39, 0.0, -0.0]                      # fp32 subnormals
    x[2, :3] = [3e38, -1e38, 1.0]
    x[3, :2] = [2.0 ** -120, 2.0 ** -126]
    x[4, :] = -0.0
    for fmt, hfmt in ((8, hip.BFP8B), (4, hip.BFP4B)):
        pd = pack_gpu(hip, dev, torch.from_numpy(x).to(dev), hfmt, (1, 32, 32), hip.F32, hip.ROW_MAJOR)
        torch.cuda.synchronize()
        want = orc.bfp_pack(x, fmt)
        assert np.array_equal(pd.cpu().numpy(), want)
        back = unpack_gpu(hip, dev, pd, hfmt, (1, 32, 32), hip.F32, hip.ROW_MAJOR)
        torch.cuda.synchronize()
        assert np.array_equal(back.cpu().numpy().view(np.uint32),
                              orc.bfp_unpack(want, (32, 32), fmt).reshape(-1).view(np.uint32))


def test_unpack_arbitrary_bytes(hip, dev, orc):
    """Every exponent/mantissa byte pattern decodes like the oracle (incl. 0x80 = -0 -> +0)."""
    rng = np.random.default_rng(9)
    for fmt, hfmt in ((8, hip.BFP8B), (4, hip.BFP4B)):
        tb = orc.bfp_tile_bytes(fmt)
        p = rng.integers(0, 256, size=16 * tb, dtype=np.uint8)
        p[:64] = np.arange(64) * 4            # low and high exponents, incl. 0 and 252
        p[tb: tb + 64] = 255 - np.arange(64)
        back = unpack_gpu(hip, dev, torch.from_numpy(p).to(dev), hfmt, (1, 128, 128), hip.F32, hip.TILE)
        torch.cuda.synchronize()
        want = orc.bfp_unpack_tiles(p, fmt)
        assert np.array_equal(back.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("fmt", [8, 4])
def test_full_size_properties(hip, dev, orc, fmt):
    """Config 2 at 8192 x 8192: every packed tile and every unpacked value against the oracle, then round-trip properties."""
    hfmt = hip.BFP8B if fmt == 8 else hip.BFP4B
    W = 7 if fmt == 8 else 3
    x = datagen.c2_outliers(8192, 8192, seed=0)
    xd = x.to(dev)
    shape = (1, 8192, 8192)
    pd = pack_gpu(hip, dev, xd, hfmt, shape, hip.F32, hip.ROW_MAJOR)
    torch.cuda.synchronize()
    tb = hip.bfp_tile_bytes(hfmt)
    assert pd.numel() == 65536 * tb
    orc.set_threads(orc.max_threads())
    try:
        want_packed = orc.bfp_pack(x.numpy(), fmt)                 # all 65 536 tiles
        want_back = orc.bfp_unpack(want_packed, (8192, 8192), fmt)
    finally:
        orc.set_threads(1)
    assert np.array_equal(pd.cpu().numpy(), want_packed)
    y = unpack_gpu(hip, dev, pd, hfmt, shape, hip.F32, hip.ROW_MAJOR).reshape(8192, 8192)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), want_back.view(np.uint32))
    del want_packed, want_back
    # idempotence: pack(unpack(pack(x))) == pack(x)
    pd2 = pack_gpu(hip, dev, y, hfmt, shape, hip.F32, hip.ROW_MAJOR)
    torch.cuda.synchronize()
    assert torch.equal(pd, pd2)
    # error bound per 16-element row: half a unit of the shared scale unless saturated
    xr, yr = xd.reshape(-1, 16), y.reshape(-1, 16)
    _, ex = torch.frexp(xr.abs().amax(dim=1))
    unit = torch.ldexp(torch.ones_like(ex, dtype=torch.float32), ex - 1 - (W - 1))[:, None]
    err = (xr - yr).abs()
    assert bool(torch.all(err <= unit))
    # (alignment bits are truncated before rounding, so a hair over half a unit is possible)
    assert bool(torch.all((err <= unit / 2 * (1 + 2.0 ** -16)) | (yr.abs() == unit * (2 ** W - 1))))
    # tilize -> untilize round trip and checksum preservation at full size
    t = torch.empty_like(xd)
    hip.call("ttm_tilize", hip.ptr(xd), hip.ptr(t), 1, 8192, 8192, 4, hip.current_stream())
    back = torch.empty_like(xd)
    hip.call("ttm_untilize", hip.ptr(t), hip.ptr(back), 1, 8192, 8192, 4, hip.current_stream())
    torch.cuda.synchronize()
    assert torch.equal(back, xd)
    assert int(t.view(torch.int32).to(torch.int64).sum()) == int(xd.view(torch.int32).to(torch.int64).sum())
    assert np.array_equal(t.reshape(-1).cpu().numpy(), orc.tilize(x.numpy()))
