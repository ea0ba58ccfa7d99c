"""Pins the oracle's tilize/untilize and scalar casts (CPU only).

Independent checks, none of which retypes the oracle's loop:
  * closed form: element (r, c) of a tile lands at ((r/16)*2 + c/16)*256 + (r%16)*16 + c%16
  * numpy reshape/transpose formulation of the same permutation
  * bijection and round trip, zero padding of ragged shapes
  * the 6-deep loop of the reference's own test (test/python/golden/d2m/test_tilize.py:45-70)
    run in pure Python on a small case
  * f16<->bf16 known answers from runtime/test/common/gtest/test_handle_float_bfloat_buffer_cast.cpp:8-46
"""
import numpy as np
import pytest


def np_tilize(x):
    b = int(np.prod(x.shape[:-2], dtype=np.int64))
    r, c = x.shape[-2:]
    return x.reshape(b, r // 32, 2, 16, c // 32, 2, 16).transpose(0, 1, 4, 2, 5, 3, 6).reshape(-1)


def test_single_tile_closed_form(orc):
    x = np.arange(1024, dtype=np.int32).reshape(32, 32)
    t = orc.tilize(x)
    for r in range(32):
        for c in range(32):
            assert t[((r // 16) * 2 + c // 16) * 256 + (r % 16) * 16 + c % 16] == x[r, c]


def test_hand_vector(orc):
    # 32x64 ramp: tile 0 face 1 row 0 starts at column 16; tile 1 starts at flat 1024 with column 32
    x = np.arange(32 * 64, dtype=np.uint16).reshape(32, 64)
    t = orc.tilize(x)
    assert list(t[:4]) == [0, 1, 2, 3]
    assert t[16] == 64            # second face row of face 0 = row 1, col 0
    assert t[256] == 16           # face 1 = cols 16..31
    assert t[512] == 16 * 64      # face 2 = rows 16..31
    assert t[768] == 16 * 64 + 16
    assert t[1024] == 32          # tile (0,1)
    assert t[2047] == 31 * 64 + 63


@pytest.mark.parametrize("shape,dtype", [((64, 96), np.float32), ((2, 3, 32, 64), np.uint16), ((96, 32), np.uint8),
                                         ((256, 512), np.uint16)])
def test_matches_numpy_formulation(orc, shape, dtype):
    rng = np.random.default_rng(1)
    x = rng.integers(0, 255, size=shape).astype(dtype)
    t = orc.tilize(x)
    assert np.array_equal(t, np_tilize(x))
    assert np.array_equal(orc.untilize(t, shape), x)


def test_reference_loop_small(orc):
    x = np.random.default_rng(2).standard_normal((64, 64)).astype(np.float32)
    out = np.zeros(x.size, dtype=np.float32)
    idx = 0
    for ty in range(2):
        for tx in range(2):
            for fy in range(2):
                for fx in range(2):
                    for dy in range(16):
                        for dx in range(16):
                            out[idx] = x[dy + ty * 32 + fy * 16, dx + tx * 32 + fx * 16]
                            idx += 1
    assert np.array_equal(orc.tilize(x), out)


def test_bijection(orc):
    x = np.arange(96 * 160, dtype=np.int32).reshape(96, 160)
    t = orc.tilize(x)
    assert sorted(t.tolist()) == list(range(96 * 160))


@pytest.mark.parametrize("shape", [(1, 1), (5, 7), (33, 31), (3, 17, 40), (1, 100)])
def test_ragged_is_zero_padded(orc, shape):
    rng = np.random.default_rng(3)
    x = rng.integers(1, 100, size=shape).astype(np.int32)
    t = orc.tilize(x)
    b, pr, pc = orc.padded_shape(shape)
    assert t.size == b * pr * pc
    xp = np.zeros((b, pr, pc), dtype=np.int32)
    xp[:, : shape[-2] if len(shape) > 1 else 1, : shape[-1]] = x.reshape(b, -1, shape[-1])
    assert np.array_equal(t, np_tilize(xp))
    assert np.array_equal(orc.untilize(t, shape), x)


def test_empty(orc):
    assert orc.tilize(np.zeros((0, 32), dtype=np.float32)).size == 0


def test_f16_bf16_known_answers(orc):
    f16 = np.array([0xBC00, 0, 0xBC00], dtype=np.uint16)
    assert orc.f16_to_bf16(f16).tolist() == [0xBF80, 0, 0xBF80]
    assert orc.bf16_to_f16(np.array([0xBF80, 0, 0xBF80], dtype=np.uint16)).tolist() == [0xBC00, 0, 0xBC00]
    # f16 max/min 65504 -> bf16 0x4780 / 0xC780 (rounds up to 65536)
    assert orc.f16_to_bf16(np.array([0xFBFF, 0x7BFF], dtype=np.uint16)).tolist() == [0xC780, 0x4780]


def test_f16_bf16_against_numpy(orc):
    import torch
    h = np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)
    f = h.view(np.float16).astype(np.float32)
    ok = np.isfinite(f)
    want = torch.from_numpy(f).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = orc.f16_to_bf16(h)
    assert np.array_equal(got[ok], want[ok])
    # bf16 -> f16, all finite bf16 whose value fits f16's range
    b = np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)
    bf = torch.from_numpy(b.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    sel = np.isfinite(bf) & (np.abs(bf) < 65520)
    want16 = bf.astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.bf16_to_f16(b)[sel], want16[sel])


def test_f32_bf16_rne(orc):
    import torch
    x = np.random.default_rng(4).standard_normal(100000).astype(np.float32) * 1e3
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(orc.f32_to_bf16(x), want)
    assert np.array_equal(orc.bf16_to_f32(want), torch.from_numpy(x).to(torch.bfloat16).float().numpy())
