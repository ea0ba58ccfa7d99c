"""The C-ABI library loads without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re


def test_header_symbols_exported(hip):
    names = [n for n, _, _ in hip.declared_functions()]
    assert len(names) >= 25
    l = ctypes.CDLL(hip.LIB_PATH)
    for n in names:
        assert hasattr(l, n), "declared but not exported: " + n


def test_every_declaration_is_parsed(hip):
    text = open(hip.HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = set(re.findall(r"\b(ttm_\w+)\s*\(", text))
    assert declared == {n for n, _, _ in hip.declared_functions()}


def test_argument_errors_without_gpu(hip):
    l = hip.lib()
    # invalid arguments are rejected on the host before any launch
    assert l.ttm_tilize(None, None, 1, 32, 32, 3, None) == 1
    assert b"elem_bytes" in l.ttm_last_error()
    assert l.ttm_bfp_pack(None, hip.F32, hip.ROW_MAJOR, None, 5, 1, 32, 32, None) == 1
    assert l.ttm_bfp_pack(None, hip.U8, hip.ROW_MAJOR, None, hip.BFP8B, 1, 32, 32, None) == 1
    assert l.ttm_set_option(b"no_such_option", 1) == 1
    assert l.ttm_bfp_tile_bytes(hip.BFP8B) == 1088 and l.ttm_bfp_tile_bytes(hip.BFP4B) == 576
    assert l.ttm_bfp_tile_bytes(hip.BF16) == -1
    # empty tensors are a no-op, not an error
    assert l.ttm_tilize(None, None, 0, 32, 32, 4, None) == 0


def test_no_oracle_in_product_path():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    pkg = os.path.join(root, "tt-mlir_amd")
    for d, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".h", ".hip")):
                src = open(os.path.join(d, f), errors="ignore").read()
                assert not re.search(r"(import|from)\s+oracle|libttm_oracle|oracle[./]|load_oracle", src), \
                    "product file reaches into the oracle: " + f


def test_buffer_extent_check_of_the_python_binding(hip):
    """The entry points take logical extents and no buffer sizes.  With check_buffers on, a pointer made by hip.ptr() must have
    the bytes behind it that the kernels touch: a [1, C] tile tensor is a full tile row of 32 rows, a reduction's result a
    full [.., rows, 1] tile per tile row.  The check raises before the library is called (no GPU needed to see it)."""
    import pytest
    import torch
    was_on = hip._check_buffers
    hip.check_buffers(True)
    try:
        C = 128256
        one_row = torch.zeros(1, C, dtype=torch.bfloat16)               # 256 KB where the kernels read 32 padded rows
        padded = torch.zeros(32, (C + 31) // 32 * 32, dtype=torch.bfloat16)
        with pytest.raises(hip.TTMError, match="tile input .argument 0. has 256512 bytes, the kernels touch 8208384"):
            hip.call("ttm_softmax_lastdim", hip.ptr(one_row), hip.ptr(padded), hip.BF16, 1, 1, C, None)
        with pytest.raises(hip.TTMError, match="tile output .argument 1."):
            hip.call("ttm_softmax_lastdim", hip.ptr(padded), hip.ptr(one_row), hip.BF16, 1, 1, C, None)
        with pytest.raises(hip.TTMError, match="tile output .*rows, 1"):
            hip.call("ttm_reduce_lastdim", 0, hip.ptr(padded), hip.ptr(torch.zeros(32, dtype=torch.bfloat16)), hip.BF16, 1, 32, C, None)
        with pytest.raises(hip.TTMError, match="weight .argument 1."):
            hip.call("ttm_rms_norm", hip.ptr(padded), hip.ptr(torch.zeros(C, dtype=torch.bfloat16)), hip.TILE, None, hip.TILE, hip.ptr(padded),
                     hip.BF16, 1, 32, C, 1e-5, None)
        with pytest.raises(hip.TTMError, match="row-major output"):
            hip.call("ttm_untilize", hip.ptr(padded), hip.ptr(one_row), 1, 32, C, 2, None)
        with pytest.raises(hip.TTMError, match="ttm_eltwise_unary: the input"):
            hip.call("ttm_eltwise_unary", 0, hip.ptr(torch.zeros(40, 50)), hip.ptr(torch.zeros(64, 64)), hip.F32, hip.TILE, 1, 40, 50, 0.0, None)
        # buffers of the right size pass the check, as does anything that is not a pointer made by ptr()
        ok = [("ttm_softmax_lastdim", (hip.ptr(padded), hip.ptr(padded), hip.BF16, 1, 32, C, None)),
              ("ttm_softmax_lastdim", (hip.ptr(padded), hip.ptr(padded), hip.BF16, 1, 1, C, None)),
              ("ttm_reduce_lastdim", (0, hip.ptr(padded), hip.ptr(torch.zeros(32 * 32, dtype=torch.bfloat16)), hip.BF16, 1, 32, C, None)),
              ("ttm_rms_norm", (hip.ptr(padded), hip.ptr(torch.zeros(C, dtype=torch.bfloat16)), hip.ROW_MAJOR, None, hip.TILE, hip.ptr(padded),
                                hip.BF16, 1, 32, C, 1e-5, None)),
              ("ttm_rms_norm", (hip.ptr(padded), hip.ptr(padded), hip.TILE, None, hip.TILE, hip.ptr(padded), hip.BF16, 1, 32, C, 1e-5, None)),
              ("ttm_tilize", (hip.ptr(torch.zeros(2, 40, 50)), hip.ptr(torch.zeros(2 * 64 * 64)), 2, 40, 50, 4, None)),
              ("ttm_eltwise_unary", (0, hip.ptr(torch.zeros(40, 50)), hip.ptr(torch.zeros(40, 50)), hip.F32, hip.ROW_MAJOR, 1, 40, 50, 0.0, None)),
              ("ttm_tilize", (None, ctypes.c_void_p(16), 0, 32, 32, 4, None)), ("ttm_sdpa", ())]
        for name, args in ok:
            hip._verify_extents(name, args)
        # block-float operands count tiles of 1088 / 576 bytes; the weights of a linear are [K, N] tiles
        a, w = torch.zeros(32 * 64, dtype=torch.bfloat16), torch.zeros(2 * 3 * 1088, dtype=torch.uint8)
        out = torch.zeros(32 * 96, dtype=torch.bfloat16)
        lin = lambda a_, w_, o_, N: ("ttm_linear", (hip.ptr(a_), hip.BF16, hip.ptr(w_), hip.BFP8B, 0, None, hip.BF16, hip.TILE, hip.ptr(o_), hip.BF16,
                                                    1, 1, 20, N, 64, 0, None))
        hip._verify_extents(*lin(a, w, out, 96))
        with pytest.raises(hip.TTMError, match="weights .*has 6528 bytes, the kernels touch 8704"):
            hip._verify_extents(*lin(a, w, torch.zeros(32 * 128, dtype=torch.bfloat16), 128))
        with pytest.raises(hip.TTMError, match="block-float output .*has 100 bytes, the kernels touch 2304"):
            hip.call("ttm_bfp_pack", hip.ptr(torch.zeros(40, 50)), hip.F32, hip.ROW_MAJOR, hip.ptr(torch.zeros(100, dtype=torch.uint8)), hip.BFP4B,
                     1, 40, 50, None)
        # off (the library's default): the call goes to the library, whose own argument check answers
        hip.check_buffers(False)
        with pytest.raises(hip.TTMError, match="elem_bytes"):
            hip.call("ttm_tilize", hip.ptr(torch.zeros(4)), hip.ptr(torch.zeros(4)), 1, 32, 32, 3, None)
    finally:
        hip.check_buffers(was_on)
