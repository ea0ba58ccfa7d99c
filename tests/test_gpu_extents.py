"""The kernel library's opt-in extent check (option "check_extents"): a call whose buffer is smaller than what the kernels
touch is refused on the host with TTM_ERR_INVALID before anything is launched.  The entry points take logical extents, and a
TILE tensor is read and written as whole 32 x 32 tiles: a [1, 128256] row handed over without its 31 padding rows would be a
GPU memory fault.  The buffers here come straight from ttm_malloc, so an allocation is exactly as large as asked for.  The
rules themselves (tt-mlir_amd/csrc/ttm_extents.h) are shared with tests/cpp/null_device.cpp and covered on the CPU by
tests/test_null_device.py."""
import ctypes

import pytest

pytestmark = pytest.mark.gpu

I64 = ctypes.c_int64


@pytest.fixture()
def checked(hip, dev):
    hip.call("ttm_set_device", 0)
    hip.set_option("check_extents", 1)
    allocs = []

    def alloc(nbytes):
        p = ctypes.c_void_p()
        hip.call("ttm_malloc", ctypes.byref(p), ctypes.c_size_t(nbytes))
        allocs.append(p)
        return p
    yield alloc
    for p in allocs:
        hip.call("ttm_free", p)
    hip.set_option("check_extents", 1)      # the suite keeps it on (conftest.py)


def refused(hip, name, *args):
    rc = getattr(hip.lib(), name)(*args)
    return rc, hip.lib().ttm_last_error().decode()


def test_short_tile_buffers_are_refused_before_the_launch(hip, checked):
    C = 128256
    Cp = (C + 31) // 32 * 32
    one_row, padded, padded2 = checked(C * 2), checked(32 * Cp * 2), checked(32 * Cp * 2)
    sm = lambda x, y, rows: refused(hip, "ttm_softmax_lastdim", x, y, hip.BF16, I64(1), I64(rows), I64(C), None)
    rc, msg = sm(one_row, padded, 1)
    assert rc == 1 and "out of bounds: ttm_softmax_lastdim: input has 256512 bytes behind it in its allocation, the kernels touch 8208384" in msg
    rc, msg = sm(padded, one_row, 1)
    assert rc == 1 and "output has 256512 bytes" in msg
    rc, msg = sm(ctypes.c_void_p(padded.value + 4096), padded2, 32)      # a view that starts inside the allocation has less room
    assert rc == 1 and "input has 8204288 bytes" in msg
    rc, msg = sm(ctypes.c_void_p(4096), padded, 1)
    assert rc == 1 and "is not device memory" in msg
    assert sm(padded, padded2, 1)[0] == 0 and sm(padded, padded2, 32)[0] == 0      # what the runtime allocates: accepted and run
    hip.call("ttm_device_sync")


def test_every_operand_of_a_linear_call_is_checked(hip, checked):
    M, K, N = 20, 96, 200
    tiles = lambda r, c: ((r + 31) // 32) * ((c + 31) // 32)
    a, w, b, out = checked(tiles(M, K) * 2048), checked(tiles(K, N) * 1088), checked(tiles(1, N) * 2048), checked(tiles(M, N) * 2048)
    small = checked(1024)                                                  # smaller than any operand of the call
    lin = lambda a_, w_, b_, o_: refused(hip, "ttm_linear", a_, hip.BF16, w_, hip.BFP8B, 0, b_, hip.BF16, hip.TILE, o_, hip.BF16, I64(1), I64(1),
                                         I64(M), I64(N), I64(K), 0, None)
    for args, what in (((small, w, b, out), "activations"), ((a, small, b, out), "weights"), ((a, w, small, out), "bias"), ((a, w, b, small), "output")):
        rc, msg = lin(*args)
        assert rc == 1 and "out of bounds: ttm_linear: " + what in msg, msg
    assert lin(a, w, None, out)[0] == 0                                    # the bias is optional
    assert lin(a, w, b, out)[0] == 0
    hip.call("ttm_device_sync")


def test_views_reductions_and_decode_operands_are_checked(hip, checked):
    buf, small = checked(64 * 64 * 2), checked(1024)
    ext, st = (I64 * 2)(64, 64), (I64 * 2)(64, 1)
    cv = lambda src, dst, base: refused(hip, "ttm_copy_view", src, I64(64), I64(64), hip.TILE, dst, I64(64), I64(64), hip.TILE, 2, 2, ext, st, I64(base), st,
                                        I64(0), None)
    assert cv(buf, buf, 0)[0] == 0
    rc, msg = cv(small, buf, 0)
    assert rc == 1 and "ttm_copy_view: source has 1024 bytes" in msg
    rc, msg = cv(buf, buf, 64)                                             # the view ends in the second matrix
    assert rc == 1 and "the kernels touch 16384" in msg
    rc, msg = cv(buf, buf, -1)
    assert rc == 1 and "negative logical offset" in msg
    rc, msg = refused(hip, "ttm_reduce_lastdim", 0, buf, small, hip.BF16, I64(1), I64(64), I64(64), None)
    assert rc == 1 and "output [.., rows, 1] has 1024 bytes" in msg and "touch 4096" in msg
    rc, msg = refused(hip, "ttm_update_cache", buf, small, small, hip.BF16, I64(1), I64(1), I64(64), I64(64), I64(1), I64(0), None)
    assert rc == 1 and "input [1, heads, users, head_dim] has 1024 bytes" in msg
    hip.call("ttm_device_sync")


def test_the_check_is_off_by_default_and_switchable(hip, checked):
    hip.set_option("check_extents", 0)
    assert hip.get_option("check_extents") == 0
    x, y = checked(64 * 64 * 4), checked(64 * 64 * 4)
    assert refused(hip, "ttm_softmax_lastdim", x, y, hip.F32, I64(1), I64(64), I64(64), None)[0] == 0     # a well-sized call either way
    hip.set_option("check_extents", 1)
    assert refused(hip, "ttm_softmax_lastdim", x, y, hip.F32, I64(1), I64(64), I64(64), None)[0] == 0
    hip.call("ttm_device_sync")
