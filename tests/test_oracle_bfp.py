"""Pins the oracle's bfp8_b / bfp4_b pack and unpack (CPU only).

The packing arithmetic lives in tt-metal, which is not part of the reference checkout: parity
with tt-metal's packer is UNPINNED.  What is pinned here is the build's own specification:
  * tile sizes 1088 / 576 bytes (lib/Dialect/TTCore/IR/TTCoreOpsTypes.cpp:1875-1887)
  * hand-worked rows (values chosen so each rule -- shared max exponent, round to nearest even,
    saturation, sign-magnitude, sign dropped at zero, nibble order -- decides one answer)
  * an independent float-arithmetic model of the encoder (floor / np.round, no bit shifts)
  * invariants: idempotence, error bounds, sign symmetry, powers of two exact, zero rows
"""
import numpy as np
import pytest


def tile_with_row(row16, face=0, r=0):
    t = np.zeros(1024, dtype=np.float32)
    t[face * 256 + r * 16: face * 256 + r * 16 + 16] = row16
    return t


def test_tile_bytes(orc):
    assert orc.bfp_tile_bytes(8) == 1088 and orc.bfp_tile_bytes(4) == 576
    x = np.zeros((64, 96), dtype=np.float32)
    assert orc.bfp_pack(x, 8).size == 6 * 1088 and orc.bfp_pack(x, 4).size == 6 * 576


def test_hand_rows_bfp8(orc):
    row = np.zeros(16, dtype=np.float32)
    row[:8] = [1.0, 0.5, -0.25, 1.9921875, 1.984375, 0.0078125, -0.00390625, 0.01171875]
    #          64    32   s|16   127.5->clamp 127  127      0.5->0 (tie to even)  -0.25->0 (sign dropped)  0.75 -> 1
    p = orc.bfp_pack_tiles(tile_with_row(row, face=2, r=5), 8)
    assert p[2 * 16 + 5] == 127                       # shared exponent = exponent of 1.x
    assert p[:64].sum() == 127                        # all other rows are zero rows -> exponent 0
    m = p[64 + 2 * 256 + 5 * 16: 64 + 2 * 256 + 5 * 16 + 16]
    assert m[:8].tolist() == [64, 32, 0x80 | 16, 127, 127, 0, 0, 1]
    assert not m[8:].any()
    back = orc.bfp_unpack_tiles(p, 8)[2 * 256 + 5 * 16: 2 * 256 + 5 * 16 + 8]
    assert back.tolist() == [1.0, 0.5, -0.25, 127 / 64, 127 / 64, 0.0, 0.0, 1 / 64]


def test_round_half_even_bfp8(orc):
    # with E=127 one unit is 2^-6; x.5 units must round to the even neighbour
    units = np.array([2.5, 3.5, 4.5, 5.5, 2.50001, 3.49999], dtype=np.float64)
    row = np.zeros(16, dtype=np.float32)
    row[0] = 1.0
    row[1:7] = (units / 64).astype(np.float32)
    p = orc.bfp_pack_tiles(tile_with_row(row), 8)
    assert p[64 + 1: 64 + 7].tolist() == [2, 4, 4, 6, 3, 3]
    # bits shifted out by the exponent alignment are truncated BEFORE rounding: 2.5 units plus
    # 4 fp32 ulps (below the 5 dropped alignment bits) is seen as an exact tie -> even
    row[1] = np.nextafter(np.float32(2.5 / 64), np.float32(1), dtype=np.float32)
    for _ in range(3):
        row[1] = np.nextafter(row[1], np.float32(1), dtype=np.float32)
    assert orc.bfp_pack_tiles(tile_with_row(row), 8)[65] == 2


def test_hand_rows_bfp4(orc):
    row = np.zeros(16, dtype=np.float32)
    row[:6] = [1.0, -1.0, 0.25, 1.75, 1.875, 0.125]
    #          4     s|4  1     7     7.5->8->clamp 7   0.5 -> 0 (tie to even)
    p = orc.bfp_pack_tiles(tile_with_row(row, face=1, r=0), 4)
    assert p[16] == 127
    m = p[64 + 128: 64 + 128 + 8]
    assert m[0] == (4 | (0xC << 4))          # even column in the low nibble
    assert m[1] == (1 | (7 << 4))
    assert m[2] == (7 | (0 << 4))
    back = orc.bfp_unpack_tiles(p, 4)[256: 256 + 6]
    assert back.tolist() == [1.0, -1.0, 0.25, 1.75, 1.75, 0.0]


def float_model_pack_row(row, W):
    """Encoder restated with float arithmetic: truncate to 24-bit fixed point at the shared
    exponent, then round half to even to W bits, saturate."""
    row = row.astype(np.float64)
    _, ex = np.frexp(np.abs(row[row != 0])) if np.any(row != 0) else (None, np.array([-125]))
    E = int(np.max(ex)) + 126 if np.any(row != 0) else 0          # biased exponent of the largest magnitude
    E = max(E, 1) if np.any(row != 0) else 0
    ulp24 = 2.0 ** (E - 127 - 23)
    q = np.floor(np.abs(row) / ulp24)                               # 24-bit fixed point, truncated
    mag = np.round(q / 2.0 ** (24 - W))                             # np.round = half to even
    mag = np.minimum(mag, 2 ** W - 1).astype(np.int64)
    sign = ((row < 0) & (mag > 0)).astype(np.int64)
    return E, (sign << W) | mag


@pytest.mark.parametrize("fmt,W", [(8, 7), (4, 3)])
def test_against_float_model(orc, fmt, W):
    rng = np.random.default_rng(7)
    x = rng.standard_normal((64, 64)).astype(np.float32)
    x[rng.random(x.shape) < 0.05] *= 100
    x[rng.random(x.shape) < 0.02] = 0
    t = orc.tilize(x)
    p = orc.bfp_pack_tiles(t, fmt)
    tb = orc.bfp_tile_bytes(fmt)
    for tile in range(4):
        for f in range(4):
            for r in range(16):
                row = t[tile * 1024 + f * 256 + r * 16:][:16]
                E, codes = float_model_pack_row(row, W)
                assert p[tile * tb + f * 16 + r] == E
                if fmt == 8:
                    got = p[tile * tb + 64 + f * 256 + r * 16:][:16].astype(np.int64)
                else:
                    b = p[tile * tb + 64 + f * 128 + r * 8:][:8].astype(np.int64)
                    got = np.stack([b & 0xF, b >> 4], axis=1).reshape(-1)
                assert np.array_equal(got, codes)


@pytest.mark.parametrize("fmt,W", [(8, 7), (4, 3)])
def test_invariants(orc, fmt, W):
    rng = np.random.default_rng(11)
    x = rng.standard_normal((128, 96)).astype(np.float32)
    x[rng.random(x.shape) < 0.01] *= 100
    p = orc.bfp_pack(x, fmt)
    y = orc.bfp_unpack(p, x.shape, fmt)
    # idempotence
    assert np.array_equal(orc.bfp_pack(y, fmt), p)
    # error bound: half a unit of the row's scale, except where saturated
    t, ty = orc.tilize(x).reshape(-1, 16), orc.tilize(y).reshape(-1, 16)
    _, ex = np.frexp(np.max(np.abs(t), axis=1))
    unit = np.ldexp(1.0, ex - 1 - (W - 1))[:, None]
    sat = np.abs(ty) == unit * (2 ** W - 1)
    # alignment bits are truncated before rounding, so a hair over half a unit is possible
    assert np.all((np.abs(t - ty) <= unit / 2 * (1 + 2.0 ** -16)) | sat)
    assert np.all(np.abs(t - ty)[sat] <= unit.repeat(16, 1)[sat])
    # sign symmetry
    yn = orc.bfp_unpack(orc.bfp_pack(-x, fmt), x.shape, fmt)
    assert np.array_equal(yn, -y)
    # decoded values never carry -0.0
    assert not np.any(np.signbit(y) & (y == 0))


def test_powers_of_two_exact_and_zero_rows(orc):
    row = np.array([2.0 ** -k for k in range(7)] + [0] * 9, dtype=np.float32)
    t = np.zeros(1024, dtype=np.float32)
    t[:16] = row
    p = orc.bfp_pack_tiles(t, 8)
    assert np.array_equal(orc.bfp_unpack_tiles(p, 8), t)
    assert p[1:64].sum() == 0 and not p[64 + 16:].any()


def test_outlier_flushes_small_values(orc):
    row = np.full(16, 0.01, dtype=np.float32)
    row[3] = 100.0
    t = np.zeros(1024, dtype=np.float32)
    t[:16] = row
    y = orc.bfp_unpack_tiles(orc.bfp_pack_tiles(t, 8), 8)[:16]
    assert y[3] == 100.0 and np.all(np.delete(y, 3) == 0.0)   # 0.01 < half a unit (0.5) at E of 100


def test_ragged_pack_matches_padded(orc):
    x = np.random.default_rng(5).standard_normal((2, 40, 50)).astype(np.float32)
    xp = np.zeros((2, 64, 64), dtype=np.float32)
    xp[:, :40, :50] = x
    for fmt in (8, 4):
        assert np.array_equal(orc.bfp_pack(x, fmt), orc.bfp_pack(xp, fmt))
        assert np.array_equal(orc.bfp_unpack(orc.bfp_pack(x, fmt), x.shape, fmt),
                              orc.bfp_unpack(orc.bfp_pack(xp, fmt), xp.shape, fmt)[:, :40, :50])
