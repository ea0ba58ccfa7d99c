"""ctypes front end of the CPU oracle (libttm_oracle.so).  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's cpu_baseline leg may import this module; the
product path never does.  Arrays are numpy; bf16 data travels as uint16 bit patterns.
Each wrapper names the reference file its C counterpart follows (see ttm_oracle.c header).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libttm_oracle.so")


def build(force=False):
    """Compile ttm_oracle.c with the committed Makefile."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE, "libttm_oracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        i64, i32, f32, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p
        sig = {
            "orc_set_threads": ([i32], None),
            "orc_max_threads": ([], i32),
            "orc_tilize": ([vp, vp, i64, i64, i64, i32], None),
            "orc_untilize": ([vp, vp, i64, i64, i64, i32], None),
            "orc_bfp_tile_bytes": ([i32], i64),
            "orc_rotary_embedding_f32": ([vp, vp, vp, vp, i64, i64, i64, i64], None),
            "orc_update_cache_f32": ([vp, vp, i64, i64, i64, i64, i64, i64], None),
            "orc_fill_cache_f32": ([vp, vp, i64, i64, i64, i64, i64], None),
            "orc_sdpa_decode_f32": ([vp, vp, vp, vp, vp, i32, vp, i64, i64, i64, i64, i64, i32, f32, i64, vp], None),
            "orc_bfp_pack_tiles": ([vp, vp, i64, i32], None),
            "orc_bfp_unpack_tiles": ([vp, vp, i64, i32], None),
            "orc_bfp_pack_rm": ([vp, vp, i64, i64, i64, i32], None),
            "orc_bfp_unpack_rm": ([vp, vp, i64, i64, i64, i32], None),
            "orc_f32_to_bf16": ([vp, vp, i64], None),
            "orc_bf16_to_f32": ([vp, vp, i64], None),
            "orc_f16_to_bf16": ([vp, vp, i64], None),
            "orc_bf16_to_f16": ([vp, vp, i64], None),
            "orc_unary_f32": ([i32, vp, vp, i64, f32], None),
            "orc_binary_f32": ([i32, vp, vp, vp, vp, vp, vp, i32], None),
            "orc_linear_f32": ([vp, vp, vp, vp, i64, i64, i64, i32, i32, i32], None),
            "orc_linear_f32_rowstream": ([vp, vp, vp, vp, i64, i64, i64, i32], None),
            "orc_bmm_f32": ([vp, vp, vp, i64, i64, i64, i64, i64, i32, i32], None),
            "orc_rmsnorm_f32": ([vp, vp, vp, vp, i64, i64, f32], None),
            "orc_softmax_f32": ([vp, vp, i64, i64, i64], None),
            "orc_reduce_f32": ([i32, vp, vp, i64, i64, i64], None),
            "orc_sdpa_f32": ([vp, vp, vp, vp, i32, vp, i64, i64, i64, i64, i64, i64, i32, f32, i64, vp], None),
        }
        for name, (args, res) in sig.items():
            fn = getattr(_lib, name)
            fn.argtypes, fn.restype = args, res
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype=None):
    a = np.ascontiguousarray(a) if dtype is None else np.ascontiguousarray(a, dtype=dtype)
    return a


def set_threads(n):
    lib().orc_set_threads(int(n))


def max_threads():
    return lib().orc_max_threads()


UNARY = dict(abs=0, ceil=1, cos=2, floor=3, gelu=4, isfinite=5, logical_not=6, neg=7, relu=8, sqrt=9,
             rsqrt=10, sigmoid=11, sin=12, reciprocal=13, sign=14, tan=15, tanh=16, atan=17, exp=18,
             erf=19, erfc=20, log=21, expm1=22, leaky_relu=23, relu6=25, silu=26, hardsigmoid=27, mish=28, acos=29,
             asin=30, asinh=31, cbrt=100, log1p=103)
BINARY = dict(add=0, multiply=1, subtract=3, eq=4, ne=5, ge=6, gt=7, le=8, lt=9, divide=10)
ACT = {None: 0, "": 0, "gelu": 1, "silu": 2, "sigmoid": 3, "relu": 4}
REDUCE = dict(sum=0, mean=1, max=2, min=3)


def _split3(shape):
    """[..., R, C] -> (batch, R, C); rank-1 tensors are one row."""
    shape = tuple(int(s) for s in shape)
    if len(shape) == 0:
        return 1, 1, 1
    if len(shape) == 1:
        return 1, 1, shape[0]
    b = 1
    for s in shape[:-2]:
        b *= s
    return b, shape[-2], shape[-1]


def padded_shape(shape):
    b, r, c = _split3(shape)
    return b, (r + 31) // 32 * 32, (c + 31) // 32 * 32


def tilize(x):
    """Row-major [..., R, C] -> flat tile-ordered array (mapping.py:3453-3495)."""
    x = _c(x)
    b, r, c = _split3(x.shape)
    _, pr, pc = padded_shape(x.shape)
    out = np.empty(b * pr * pc, dtype=x.dtype)
    lib().orc_tilize(_p(x), _p(out), b, r, c, x.dtype.itemsize)
    return out


def untilize(t, shape):
    """Flat tile-ordered array -> row-major array of `shape` (mapping.py:3498-3549)."""
    t = _c(t)
    b, r, c = _split3(shape)
    out = np.empty(shape, dtype=t.dtype)
    lib().orc_untilize(_p(t), _p(out), b, r, c, t.dtype.itemsize)
    return out


def bfp_tile_bytes(fmt):
    return int(lib().orc_bfp_tile_bytes(fmt))


def bfp_pack_tiles(tiled_f32, fmt):
    t = _c(tiled_f32, np.float32).reshape(-1)
    assert t.size % 1024 == 0
    n = t.size // 1024
    out = np.empty(n * bfp_tile_bytes(fmt), dtype=np.uint8)
    lib().orc_bfp_pack_tiles(_p(t), _p(out), n, fmt)
    return out


def bfp_unpack_tiles(packed, fmt):
    p = _c(packed, np.uint8).reshape(-1)
    n = p.size // bfp_tile_bytes(fmt)
    out = np.empty(n * 1024, dtype=np.float32)
    lib().orc_bfp_unpack_tiles(_p(p), _p(out), n, fmt)
    return out


def bfp_pack(x_f32, fmt):
    """Row-major fp32 [..., R, C] -> packed bfp tiles (tilize fused, zero padded)."""
    x = _c(x_f32, np.float32)
    b, r, c = _split3(x.shape)
    _, pr, pc = padded_shape(x.shape)
    out = np.empty(b * (pr // 32) * (pc // 32) * bfp_tile_bytes(fmt), dtype=np.uint8)
    lib().orc_bfp_pack_rm(_p(x), _p(out), b, r, c, fmt)
    return out


def bfp_unpack(packed, shape, fmt):
    p = _c(packed, np.uint8).reshape(-1)
    b, r, c = _split3(shape)
    out = np.empty(shape, dtype=np.float32)
    lib().orc_bfp_unpack_rm(_p(p), _p(out), b, r, c, fmt)
    return out


def f32_to_bf16(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_f32_to_bf16(_p(x), _p(out), x.size)
    return out


def bf16_to_f32(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib().orc_bf16_to_f32(_p(h), _p(out), h.size)
    return out


def f16_to_bf16(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, dtype=np.uint16)
    lib().orc_f16_to_bf16(_p(h), _p(out), h.size)
    return out


def bf16_to_f16(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, dtype=np.uint16)
    lib().orc_bf16_to_f16(_p(h), _p(out), h.size)
    return out


def round_bf16(x):
    """f32 -> bf16 -> f32 (the CPU path's final cast back, HoistCPUOps.cpp:219-245)."""
    return bf16_to_f32(f32_to_bf16(x))


def unary(op, x, param=0.0):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    lib().orc_unary_f32(UNARY[op], _p(x), _p(out), x.size, float(param))
    return out


def binary(op, a, b):
    a, b = _c(a, np.float32), _c(b, np.float32)
    oshape = np.broadcast_shapes(a.shape, b.shape)
    rank = max(len(oshape), 1)
    pad = lambda s: np.array((1,) * (rank - len(s)) + tuple(s), dtype=np.int64)
    out = np.empty(oshape, dtype=np.float32)
    lib().orc_binary_f32(BINARY[op], _p(a), _p(pad(a.shape)), _p(b), _p(pad(b.shape)), _p(out),
                         _p(pad(oshape)), rank)
    return out


def linear(a, b, bias=None, act=None, transpose_a=False, transpose_b=False, rowstream=False):
    """act(a @ b + bias), 2-D operands, f32 (TTIRToLinalg.cpp:1647-1912, mapping.py:7749-7797)."""
    a, b = _c(a, np.float32), _c(b, np.float32)
    M, K = (a.shape[1], a.shape[0]) if transpose_a else a.shape
    N = b.shape[0] if transpose_b else b.shape[1]
    bias = None if bias is None else _c(bias, np.float32).reshape(-1)
    out = np.empty((M, N), dtype=np.float32)
    if rowstream:
        assert not transpose_a and not transpose_b
        lib().orc_linear_f32_rowstream(_p(a), _p(b), _p(bias), _p(out), M, N, K, ACT[act])
    else:
        lib().orc_linear_f32(_p(a), _p(b), _p(bias), _p(out), M, N, K, int(transpose_a), int(transpose_b),
                             ACT[act])
    return out


def matmul(a, b, transpose_a=False, transpose_b=False):
    """Batched matmul; b may have a single batch (TTIRToLinalg.cpp:318-572)."""
    a, b = _c(a, np.float32), _c(b, np.float32)
    if a.ndim == 2 and b.ndim == 2:
        return linear(a, b, None, None, transpose_a, transpose_b)
    ba, ra, ca = _split3(a.shape)
    bb, rb, cb = _split3(b.shape)
    M, K = (ca, ra) if transpose_a else (ra, ca)
    N = rb if transpose_b else cb
    assert bb in (1, ba)
    out = np.empty(tuple(a.shape[:-2]) + (M, N), dtype=np.float32)
    lib().orc_bmm_f32(_p(a), _p(b), _p(out), ba, bb, M, N, K, int(transpose_a), int(transpose_b))
    return out


def rms_norm(x, weight=None, bias=None, eps=1e-5):
    x = _c(x, np.float32)
    cols = x.shape[-1]
    w = None if weight is None else _c(weight, np.float32).reshape(-1)
    b = None if bias is None else _c(bias, np.float32).reshape(-1)
    out = np.empty_like(x)
    lib().orc_rmsnorm_f32(_p(x), _p(w), _p(b), _p(out), x.size // cols, cols, float(eps))
    return out


def _odi(shape, dim):
    dim = dim % len(shape)
    outer = int(np.prod(shape[:dim], dtype=np.int64))
    inner = int(np.prod(shape[dim + 1:], dtype=np.int64))
    return outer, int(shape[dim]), inner


def softmax(x, dim=-1):
    x = _c(x, np.float32)
    o, d, i = _odi(x.shape, dim)
    out = np.empty_like(x)
    lib().orc_softmax_f32(_p(x), _p(out), o, d, i)
    return out


def reduce(op, x, dim=-1, keepdim=False):
    x = _c(x, np.float32)
    o, d, i = _odi(x.shape, dim)
    dim = dim % x.ndim
    oshape = list(x.shape)
    oshape[dim] = 1
    out = np.empty(oshape, dtype=np.float32)
    lib().orc_reduce_f32(REDUCE[op], _p(x), _p(out), o, d, i)
    return out if keepdim else out.reshape([s for k, s in enumerate(x.shape) if k != dim])


def sdpa(q, k, v, mask=None, is_causal=False, scale=None, sliding_window=None, attention_sink=None):
    """attention_sink: the TTNN operand, any shape holding one value per query head ([1, Hq, 1, 1])."""
    q, k, v = _c(q, np.float32), _c(k, np.float32), _c(v, np.float32)
    B, Hq, Sq, D = q.shape
    _, Hkv, Sk, _ = k.shape
    mh = 1
    if mask is not None:
        mask = _c(mask, np.float32)
        mh = mask.shape[1]
        if mask.shape[0] == 1 and B > 1:               # one mask shared by the batch
            mask = _c(np.broadcast_to(mask, (B,) + mask.shape[1:]))
    out = np.empty_like(q)
    sink = None if attention_sink is None else _c(attention_sink, np.float32).reshape(Hq)
    lib().orc_sdpa_f32(_p(q), _p(k), _p(v), _p(mask), mh, _p(out), B, Hq, Hkv, Sq, Sk, D, int(is_causal),
                       float(scale) if scale else 0.0, -1 if sliding_window is None else int(sliding_window), _p(sink))
    return out


def rotary_embedding(x, cos, sin, token_index=None):
    """x [..., rows, D], cos / sin [..., cache_rows, D] (leading 1s dropped)."""
    x = _c(x, np.float32)
    D = x.shape[-1]
    cos, sin = _c(cos, np.float32).reshape(-1, D), _c(sin, np.float32).reshape(-1, D)
    rows = x.shape[-2]
    out = np.empty_like(x)
    lib().orc_rotary_embedding_f32(_p(x), _p(cos), _p(sin), _p(out), x.size // (rows * D), rows, D,
                                   -1 if token_index is None else int(token_index))
    return out


def update_cache(cache, inp, update_index, batch_offset=0):
    cache, inp = _c(cache, np.float32).copy(), _c(inp, np.float32)
    U, H, S, D = cache.shape
    lib().orc_update_cache_f32(_p(cache), _p(inp), H, S, D, inp.shape[2], int(update_index), int(batch_offset))
    return cache


def fill_cache(cache, inp, batch_offset=0):
    cache, inp = _c(cache, np.float32).copy(), _c(inp, np.float32)
    U, H, S, D = cache.shape
    lib().orc_fill_cache_f32(_p(cache), _p(inp), H, S, D, inp.shape[2], int(batch_offset))
    return cache


def paged_update_cache(cache, inp, update_index, page_table=None, share_cache=False):
    """tools/golden/mapping.py:8926-8963 with the operand shapes of the TTNN op (lib/Dialect/TTNN/IR/TTNNOps.cpp:4719-4820):
    cache [blocks, heads, block_size, dim], inp [1, users, heads, dim], update_index [users], page_table [users, pages].
    cache[page_table[u, p // block_size], :, p % block_size, :] = inp[0, u] with p = update_index[u]; without a page table
    user u owns cache entry u (entry 0 when the cache is shared).  Out-of-range positions, pages and blocks write nothing
    (the golden clamps them instead; valid inputs never get there)."""
    cache, inp = _c(cache, np.float32).copy(), _c(inp, np.float32)
    blocks, _, bs, _ = cache.shape
    for u in range(inp.shape[1]):
        p = int(update_index[u])
        if p < 0:
            continue
        if page_table is not None:
            page = p // bs
            if page >= page_table.shape[1]:
                continue
            blk, off = int(page_table[u, page]), p % bs
        else:
            if p >= bs:
                continue
            blk, off = (0 if share_cache else u), p
        if 0 <= blk < blocks:
            cache[blk, :, off, :] = inp[0, u]
    return cache


def paged_fill_cache(cache, inp, page_table, batch_idx=None):
    """tools/golden/mapping.py:8966-9008: cache [blocks, heads, block_size, dim], inp [batch, heads, seq, dim];
    cache[page_table[row(b), s // block_size], :, s % block_size, :] = inp[b, :, s, :], row(b) = batch_idx[b] or b."""
    cache, inp = _c(cache, np.float32).copy(), _c(inp, np.float32)
    blocks, _, bs, _ = cache.shape
    for b in range(inp.shape[0]):
        row = int(batch_idx[b]) if batch_idx is not None else b
        if not 0 <= row < page_table.shape[0]:
            continue
        for sq in range(inp.shape[2]):
            page = sq // bs
            if page >= page_table.shape[1]:
                continue
            blk = int(page_table[row, page])
            if 0 <= blk < blocks:
                cache[blk, :, sq % bs, :] = inp[b, :, sq, :]
    return cache


def sdpa_decode(q, k, v, cur_pos=None, mask=None, is_causal=True, scale=None, sliding_window=None, attention_sink=None):
    """attention_sink: the op's [H, 32] operand (column 0 is read) or one value per head."""
    q, k, v = _c(q, np.float32), _c(k, np.float32), _c(v, np.float32)
    _, B, H, D = q.shape
    _, Hkv, S, _ = k.shape
    cp = None if cur_pos is None else np.ascontiguousarray(cur_pos, dtype=np.int32)
    mh = 1
    if mask is not None:
        mask = _c(mask, np.float32)
        mh = mask.shape[2]
        if mask.shape[0] == 1 and B > 1:               # one mask shared by the users
            mask = _c(np.broadcast_to(mask, (B,) + mask.shape[1:]))
    out = np.empty_like(q)
    sink = None
    if attention_sink is not None:
        sink = _c(attention_sink, np.float32)
        sink = _c(sink[:, 0] if sink.ndim == 2 else sink.reshape(H), np.float32)
    lib().orc_sdpa_decode_f32(_p(q), _p(k), _p(v), _p(cp), _p(mask), mh, _p(out), B, H, Hkv, S, D, int(is_causal),
                              float(scale) if scale else 0.0, -1 if sliding_window is None else int(sliding_window), _p(sink))
    return out


# ---- the ops around a decoder layer (embedding in front, argmax behind, mask construction beside it).  Each is the
# library routine the reference's golden calls, on numpy arrays: nothing here has arithmetic of its own to get wrong
# except the index conventions, which tests/test_oracle_math.py checks against torch.
def where(cond, a, b):
    """tools/golden/mapping.py:5579-5586 (torch.where); cond != 0 selects a."""
    return np.where(np.asarray(cond) != 0, a, b)


def embedding(indices, weight):
    """tools/golden/mapping.py:2900-2912: rows of the [.., vocab, dim] table, indices clamped to [0, vocab - 1]."""
    w = np.asarray(weight)
    w = w.reshape(w.shape[-2], w.shape[-1])
    idx = np.clip(np.asarray(indices).astype(np.int64), 0, w.shape[0] - 1)
    return w[idx]


def argmax(x, dim=None, keep_dim=False):
    """tools/golden/mapping.py:5222-5265 (torch.argmax): first index of the largest element, over `dim` or the whole tensor."""
    x = np.asarray(x)
    if dim is None:
        r = np.argmax(x.reshape(-1))
        return np.full((1,) * x.ndim if keep_dim else (), r, dtype=np.int32)
    r = np.argmax(x, axis=dim).astype(np.int32)
    return np.expand_dims(r, dim) if keep_dim else r


def arange(start, end, step=1, dtype=np.float32):
    """tools/golden/mapping.py:4269-4290: torch.arange in float32, then the cast."""
    return np.arange(start, end, step, dtype=np.float32).astype(dtype)


def repeat(x, repeats):
    """tools/golden/mapping.py:4259-4266 (Tensor.repeat = numpy tile with one count per dimension)."""
    return np.tile(np.asarray(x), tuple(int(r) for r in repeats))


def binary_composite(name, a, b):
    """maximum / minimum / remainder / pow / atan2 as the goldens take them from torch (tools/golden/mapping.py:4493-4570,
    5516-5530): NaN propagates through maximum and minimum, remainder has the sign of the divisor."""
    a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
    with np.errstate(all="ignore"):
        return {"maximum": np.maximum, "minimum": np.minimum, "remainder": np.mod, "pow": np.power,
                "atan2": np.arctan2}[name](a, b).astype(np.float32)


def clamp(x, lo, hi):
    """tools/golden/mapping.py:5267-5276 (torch.clamp with scalar bounds; NaN stays NaN)."""
    x = np.asarray(x, np.float32)
    return np.where(np.isnan(x), x, np.minimum(np.maximum(x, np.float32(lo)), np.float32(hi))).astype(np.float32)


def chunked_sdpa(q, k_pages, v_pages, page_table, chunk_start, scale=None):
    """Chunked prefill over a paged cache (tools/golden/mapping.py:8847-8913): q [B, H, Sq, D]; pages [blocks, Hkv, block, D];
    page_table [B, pages_per_user]; query row j stands at position chunk_start + j and sees keys [0, chunk_start + j].  The
    pages are unpaged with the table (entries clamped into range, as the golden does), the band is written as an additive
    mask and the prefill attention of this module does the rest."""
    q, kp, vp = _c(q, np.float32), _c(k_pages, np.float32), _c(v_pages, np.float32)
    B, H, Sq, D = q.shape
    blocks, Hkv, block, _ = kp.shape
    pt = np.clip(np.asarray(page_table, dtype=np.int64), 0, blocks - 1)
    pages = pt.shape[-1]
    Sk = pages * block
    unpage = lambda c: _c(c[pt.reshape(-1)].reshape(B, pages, Hkv, block, D).transpose(0, 2, 1, 3, 4).reshape(B, Hkv, Sk, D))
    col = np.arange(Sk)[None, :]
    row = (int(chunk_start) + np.arange(Sq))[:, None]
    mask = np.where(col <= row, 0.0, -np.inf).astype(np.float32)[None, None]
    return sdpa(q, unpage(kp), unpage(vp), mask=mask, is_causal=False, scale=scale)


def rotary_embedding_llama(x, cos, sin, trans_mat):
    """out = x * cos + (x T) * sin with the 32 x 32 matrix T applied to every 32-column tile of the last dim
    (::ttnn::experimental::rotary_embedding_llama as called from runtime/lib/ttnn/operations/transformer/
    rotary_embedding_llama.cpp:11-34; the op has no golden in the reference).  x [.., R, D]; cos / sin broadcast
    against it; f32 arithmetic, as the CPU path computes."""
    x = _c(x, np.float32)
    T = _c(trans_mat, np.float32).reshape(32, 32)
    xt = x.reshape(x.shape[:-1] + (x.shape[-1] // 32, 32))
    rot = np.einsum("...tj,jc->...tc", xt, T).reshape(x.shape).astype(np.float32)
    return (x * np.asarray(cos, dtype=np.float32) + rot * np.asarray(sin, dtype=np.float32)).astype(np.float32)
