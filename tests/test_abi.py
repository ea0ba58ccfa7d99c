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
