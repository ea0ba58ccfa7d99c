"""The oracle and the runtime's host-side casts against the known answers the reference's own tests hold
(tests/golden/reference_known_answers.json; each block names its reference file)."""
import json
import os

import numpy as np
import pytest

from ttmlir_amd import hip, runtime as rt

DT = rt.DataType
G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))


def test_float_bfloat_casts():
    for case in G["f16_to_bf16"]["cases"]:
        src = np.array(case["in_bits"], dtype=np.uint16).view(np.float16)
        assert rt.buffer_cast(src, DT.Float16, DT.BFloat16).tolist() == case["out_bits"]
    for case in G["bf16_to_f16"]["cases"]:
        src = np.array(case["in_bits"], dtype=np.uint16)
        assert rt.buffer_cast(src, DT.BFloat16, DT.Float16).view(np.uint16).tolist() == case["out_bits"]


def test_integer_casts_saturate():
    np_of = {"Int64": np.int64, "UInt64": np.uint64, "Int16": np.int16, "UInt16": np.uint16, "Int8": np.int8}
    for case in G["integer_saturation"]["cases"]:
        src = np.array(case["in"], dtype=np_of[case["from"]])
        assert rt.buffer_cast(src, getattr(DT, case["from"]), getattr(DT, case["to"])).tolist() == case["out"]


def test_gelu_doc_example(orc):
    g = G["gelu_doc_example"]
    got = orc.unary("gelu", np.array(g["in"], dtype=np.float32))
    assert np.max(np.abs(got - np.array(g["out"]))) <= g["abs_tol"]


def test_tilize_positions(orc):
    x = np.arange(1024, dtype=np.int32).reshape(32, 32)
    t = orc.tilize(x)
    for case in G["tilize_element_position"]["cases"]:
        assert t[case["pos"]] == x[case["r"], case["c"]]


def test_size_contract():
    assert hip.bfp_tile_bytes(hip.BFP8B) == G["bfp_tile_bytes"]["bfp8"] and hip.bfp_tile_bytes(hip.BFP4B) == G["bfp_tile_bytes"]["bfp4"]
