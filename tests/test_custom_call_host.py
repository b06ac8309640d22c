"""Operator contract, host side only (mirrors Tests/MetalHLOCoreTests/CustomCallTests.swift:14-155):
registry contents, backend_config parsing semantics and operand-count errors."""
import pytest

from metalhlo_amd import custom_call as cc
from metalhlo_amd.custom_call import BackendConfigParser as P


def test_registry_contents():
    reg = cc.shared
    for t in ["fused_scaled_dot_product_attention", "fused_layer_norm", "fused_rms_norm",
              "fused_matmul_bias_activation", "fused_softmax", "fused_gelu", "fused_ffn", "fused_rope",
              "fused_elementwise", "fused_batch_norm", "fused_depth_attention"]:
        assert reg.has_handler(t)
    assert not reg.has_handler("unknown_target")
    for t in cc.NOT_ON_PATH:
        with pytest.raises(cc.UnsupportedTarget):
            reg.emit(t, [], "")


def test_backend_config_parser_semantics():
    assert P.parse("") == {} and P.parse("not json") == {} and P.parse("[1,2]") == {}
    cfg = P.parse('{"scale": 0.125, "has_mask": true, "axis": -1, "axes": [-1], "activation": "gelu", "n": 3, "one": 1}')
    assert P.get_float(cfg, "scale", 1.0) == 0.125
    assert P.get_float(cfg, "n", 1.0) == 3.0            # int accepted as float
    assert P.get_float(cfg, "missing", 7.5) == 7.5
    assert P.get_float(cfg, "activation", 7.5) == 7.5   # wrong type -> default
    assert P.get_int(cfg, "axis", 0) == -1 and P.get_int(cfg, "scale", 9) == 0   # double truncates
    assert P.get_bool(cfg, "has_mask", False) is True
    assert P.get_bool(cfg, "one", False) is True        # int != 0
    assert P.get_bool(cfg, "missing", True) is True
    assert P.get_string(cfg, "activation", "none") == "gelu" and P.get_string(cfg, "n", "none") == "none"
    assert P.get_int_array(cfg, "axes", [0]) == [-1] and P.get_int_array(cfg, "axis", [5]) == [5]


def test_operand_count_errors_before_any_launch():
    reg = cc.shared
    with pytest.raises(cc.InvalidInputCount) as e:
        reg.emit("fused_scaled_dot_product_attention", [None, None], "")
    assert (e.value.expected, e.value.got) == (3, 2)
    with pytest.raises(cc.InvalidInputCount):
        reg.emit("fused_layer_norm", [None, None], "")
    with pytest.raises(cc.InvalidInputCount):
        reg.emit("fused_rms_norm", [None], "")
    with pytest.raises(cc.InvalidInputCount):
        reg.emit("fused_softmax", [], "")
    with pytest.raises(cc.InvalidInputCount):
        reg.emit("fused_matmul_bias_activation", [None], "")
