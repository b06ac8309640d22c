"""mhlo_* C API without a GPU (METALHLO_ALLOW_NO_DEVICE=1 gives a host-only client):
symbols, defaults, NULL / parse / unsupported-op error codes and the type queries.
Restates the host-only parts of Tests/MetalHLOTests/CAPITests.swift:15-689."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
os.environ["METALHLO_ALLOW_NO_DEVICE"] = "1"

from metalhlo_amd import capi  # noqa: E402

ADD = """
module @add {
  func.func @main(%arg0: tensor<2x3xf32>, %arg1: tensor<2x3xf32>) -> (tensor<2x3xf32>) {
    %0 = stablehlo.add %arg0, %arg1 : tensor<2x3xf32>
    return %0 : tensor<2x3xf32>
  }
}
"""


@pytest.fixture(scope="module")
def lib():
    return capi.load()


@pytest.fixture()
def client(lib):
    c = C.c_void_p()
    assert lib.mhlo_client_create(C.byref(c)) == 0
    yield c
    lib.mhlo_client_destroy(c)


def test_exports_every_declared_symbol(lib):
    src = open(os.path.join(ROOT, "include", "metalhlo.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    names = sorted(set(re.findall(r"\b(mhlo_[a-z0-9_]+)\s*\(", src)))
    assert len(names) == 34        # the reference's 31 + mhlo_ext_executable_ops, _plan and _profile
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(capi.SIGNATURES) == names


def test_version_sizes_defaults(lib):
    assert lib.mhlo_version() == b"0.2.0"
    sizes = {0: 2, 1: 4, 2: 8, 3: 2, 4: 0, 5: 1, 6: 2, 7: 4, 8: 8, 9: 1, 10: 2, 11: 4, 12: 8}
    for et, sz in sizes.items():
        assert lib.mhlo_element_type_size(et) == sz
    cfg = capi.CompileConfig(9, False, True, 3)
    lib.mhlo_compile_config_init(C.byref(cfg))
    assert (cfg.optimization_level, cfg.enable_caching, cfg.enable_debug_info, cfg.device_policy) == (2, True, False, 0)
    lib.mhlo_compile_config_init(None)       # NULL is ignored
    assert lib.mhlo_ane_available() is False


def test_null_arguments_are_invalid_argument(lib, client):
    exe = C.c_void_p()
    assert lib.mhlo_client_create(None) == 10 and b"out_client is null" in lib.mhlo_get_last_error()
    assert lib.mhlo_compile(None, ADD.encode(), C.byref(exe)) == 10 and b"client is null" in lib.mhlo_get_last_error()
    assert lib.mhlo_compile(client, None, C.byref(exe)) == 10 and b"mlir_text is null" in lib.mhlo_get_last_error()
    assert lib.mhlo_compile(client, ADD.encode(), None) == 10 and b"out_executable is null" in lib.mhlo_get_last_error()
    assert lib.mhlo_execute(None, None, 0, None, None) == 10
    assert lib.mhlo_buffer_to_host(None, None, 0) == 10
    assert lib.mhlo_executable_get_stats(None, None) == 10
    lib.mhlo_clear_error()
    assert lib.mhlo_get_last_error() is None
    assert lib.mhlo_executable_input_count(None) == 0 and lib.mhlo_buffer_rank(None) == 0


def test_compile_and_type_queries(lib, client):
    exe = C.c_void_p()
    assert lib.mhlo_compile(client, ADD.encode(), C.byref(exe)) == 0, lib.mhlo_get_last_error()
    assert lib.mhlo_get_last_error() is None
    assert lib.mhlo_executable_input_count(exe) == 2 and lib.mhlo_executable_output_count(exe) == 1
    shape = (C.c_int64 * 4)()
    rank, et = C.c_int32(), C.c_int()
    assert lib.mhlo_executable_input_type(exe, 1, shape, C.byref(rank), C.byref(et)) == 0
    assert (rank.value, et.value, shape[0], shape[1]) == (2, 1, 2, 3)
    assert lib.mhlo_executable_output_type(exe, 0, None, C.byref(rank), None) == 0 and rank.value == 2
    assert lib.mhlo_executable_input_type(exe, 5, None, None, None) == 10
    st = capi.ExecutionStats()
    assert lib.mhlo_executable_get_stats(exe, C.byref(st)) == 0 and st.execution_count == 0
    cfg = capi.CompileConfig()
    lib.mhlo_compile_config_init(C.byref(cfg))
    cfg.optimization_level = 3
    exe2 = C.c_void_p()
    assert lib.mhlo_compile_with_config(client, ADD.encode(), C.byref(cfg), C.byref(exe2)) == 0
    assert lib.mhlo_compile_with_config(client, ADD.encode(), None, C.byref(exe2)) == 0     # NULL config = defaults
    text = ADD.encode() + b"garbage after the length"
    assert lib.mhlo_compile_n(client, text, len(ADD.encode()), C.byref(exe2)) == 0
    lib.mhlo_executable_destroy(exe)


def test_error_codes(lib, client):
    exe = C.c_void_p()
    assert lib.mhlo_compile(client, b"this is not mlir", C.byref(exe)) == 3
    assert b"Parse failed" in lib.mhlo_get_last_error()
    bad = ADD.replace("stablehlo.add %arg0, %arg1", "stablehlo.add %arg0, %nope")
    assert lib.mhlo_compile(client, bad.encode(), C.byref(exe)) == 3 and b"undefined value" in lib.mhlo_get_last_error()
    unsup = ADD.replace("stablehlo.add", "stablehlo.atan2")
    assert lib.mhlo_compile(client, unsup.encode(), C.byref(exe)) == 4
    cc = """func.func @main(%a: tensor<4xf32>) -> tensor<4xf32> {
      %0 = stablehlo.custom_call @fused_conv_bias_act(%a) {backend_config = "{}"} : (tensor<4xf32>) -> tensor<4xf32>
      return %0 : tensor<4xf32> }"""
    assert lib.mhlo_compile(client, cc.encode(), C.byref(exe)) == 4 and b"fused_conv_bias_act" in lib.mhlo_get_last_error()
    few = """func.func @main(%a: tensor<4x8xf32>) -> tensor<4x8xf32> {
      %0 = stablehlo.custom_call @fused_layer_norm(%a) {backend_config = "{}"} : (tensor<4x8xf32>) -> tensor<4x8xf32>
      return %0 : tensor<4x8xf32> }"""
    assert lib.mhlo_compile(client, few.encode(), C.byref(exe)) == 3 and b"expected 3, got 1" in lib.mhlo_get_last_error()
    emb = """func.func @main(%i: tensor<2x8xi32>, %t: tensor<10x16xf32>, %p: tensor<12x16xf32>) -> tensor<2x8x16xbf16> {
      %0 = stablehlo.custom_call @fused_token_embedding(%i, %t, %p) {backend_config = "{\\"first_position\\": FIRST}"} : (tensor<2x8xi32>, tensor<10x16xf32>, tensor<12x16xf32>) -> tensor<2x8x16xbf16>
      return %0 : tensor<2x8x16xbf16> }"""
    assert lib.mhlo_compile(client, emb.replace("FIRST", "4").encode(), C.byref(exe)) == 0
    lib.mhlo_executable_destroy(exe)
    assert lib.mhlo_compile(client, emb.replace("FIRST", "5").encode(), C.byref(exe)) == 3 and b"positions outside" in lib.mhlo_get_last_error()
    assert lib.mhlo_compile(client, emb.replace("FIRST", "0").replace("2x8xi32", "2x8xi64").encode(), C.byref(exe)) == 3
    # without a device: buffers and execution report NO_DEVICE, nothing crashes
    buf = C.c_void_p()
    shape = (C.c_int64 * 1)(4)
    data = (C.c_float * 4)(1, 2, 3, 4)
    assert lib.mhlo_buffer_create(client, data, 16, shape, 1, 1, C.byref(buf)) == 1
    assert lib.mhlo_buffer_create(client, data, 8, shape, 1, 1, C.byref(buf)) == 6      # data_size too small
    assert lib.mhlo_buffer_create(client, None, 16, shape, 1, 1, C.byref(buf)) == 10


PARSE_CASES = {
    "generic_form": """func.func @main(%arg0: tensor<2x3xf32>) -> tensor<3x2xf32> {
        %0 = "stablehlo.transpose"(%arg0) {permutation = array<i64: 1, 0>} : (tensor<2x3xf32>) -> tensor<3x2xf32>
        return %0 : tensor<3x2xf32> }""",
    "dot_general_attr": """func.func @main(%l: tensor<2x3x4xf32>, %r: tensor<2x4x5xf32>) -> (tensor<2x3x5xf32>) {
        %0 = stablehlo.dot_general %l, %r, #stablehlo.dot<lhs_batching_dimensions = [0], rhs_batching_dimensions = [0], lhs_contracting_dimensions = [2], rhs_contracting_dimensions = [1]> : (tensor<2x3x4xf32>, tensor<2x4x5xf32>) -> tensor<2x3x5xf32>
        return %0 : tensor<2x3x5xf32> }""",
    "dot_general_pretty": """func.func @main(%l: tensor<2x3x4xbf16>, %r: tensor<2x4x5xbf16>) -> tensor<2x3x5xbf16> {
        %0 = stablehlo.dot_general %l, %r, batching_dims = [0] x [0], contracting_dims = [2] x [1], precision = [DEFAULT, DEFAULT] : (tensor<2x3x4xbf16>, tensor<2x4x5xbf16>) -> tensor<2x3x5xbf16>
        return %0 : tensor<2x3x5xbf16> }""",
    "reduce_both_spellings": """func.func @main(%x: tensor<4x8xf32>) -> tensor<4xf32> {
        %c = stablehlo.constant dense<0.0> : tensor<f32>
        %m = stablehlo.constant dense<0xFF800000> : tensor<f32>
        %0 = stablehlo.reduce(%x init: %c) applies stablehlo.add across dimensions = [1] : (tensor<4x8xf32>, tensor<f32>) -> tensor<4xf32>
        %1 = stablehlo.reduce %x, %m applies stablehlo.maximum across dimensions = [1] : (tensor<4x8xf32>, tensor<f32>) -> tensor<4xf32>
        %2 = stablehlo.add %0, %1 : tensor<4xf32>
        return %2 : tensor<4xf32> }""",
    "reduce_region": """func.func @main(%x: tensor<4x8xf32>) -> tensor<4xf32> {
        %c = stablehlo.constant dense<0.0> : tensor<f32>
        %0 = stablehlo.reduce(%x init: %c) across dimensions = [1] : (tensor<4x8xf32>, tensor<f32>) -> tensor<4xf32>
         reducer(%a: tensor<f32>, %b: tensor<f32>)  {
          %s = stablehlo.add %a, %b : tensor<f32>
          stablehlo.return %s : tensor<f32>
        }
        return %0 : tensor<4xf32> }""",
    "constants_iota_compare_select": """func.func @main(%x: tensor<2x2xf32>) -> tensor<2x2xf32> {
        %c = stablehlo.constant dense<[[1.0, -2.5], [3.0e+00, 4.0]]> : tensor<2x2xf32>
        %i = stablehlo.iota dim = 1 : tensor<2x2xi32>
        %j = stablehlo.iota dim = 0 : tensor<2x2xi32>
        %p = stablehlo.compare GT, %i, %j, SIGNED : (tensor<2x2xi32>, tensor<2x2xi32>) -> tensor<2x2xi1>
        %0 = stablehlo.select %p, %c, %x : tensor<2x2xi1>, tensor<2x2xf32>
        return %0 : tensor<2x2xf32> }""",
    "custom_calls": """func.func @main(%q: tensor<1x4x128x64xbf16>, %k: tensor<1x4x128x64xbf16>, %v: tensor<1x4x128x64xbf16>, %g: tensor<64xbf16>) -> tensor<1x4x128x64xbf16> {
        %0 = stablehlo.custom_call @fused_scaled_dot_product_attention(%q, %k, %v) {backend_config = "{\\"scale\\": 0.125, \\"is_causal\\": true}"} : (tensor<1x4x128x64xbf16>, tensor<1x4x128x64xbf16>, tensor<1x4x128x64xbf16>) -> tensor<1x4x128x64xbf16>
        %1 = stablehlo.custom_call @fused_rms_norm(%0, %g) {backend_config = "{\\"eps\\": 1e-6, \\"axes\\": [-1]}"} : (tensor<1x4x128x64xbf16>, tensor<64xbf16>) -> tensor<1x4x128x64xbf16>
        return %1 : tensor<1x4x128x64xbf16> }""",
    "slice_broadcast_convert_reshape": """func.func @main(%x: tensor<4x6xf32>, %b: tensor<3xf32>) -> tensor<2x3xbf16> {
        %s = stablehlo.slice %x [1:3, 0:6:2] : (tensor<4x6xf32>) -> tensor<2x3xf32>
        %bb = stablehlo.broadcast_in_dim %b, dims = [1] : (tensor<3xf32>) -> tensor<2x3xf32>
        %a = stablehlo.add %s, %bb : tensor<2x3xf32>
        %r = stablehlo.reshape %a : (tensor<2x3xf32>) -> tensor<6xf32>
        %r2 = stablehlo.reshape %r : (tensor<6xf32>) -> tensor<2x3xf32>
        %c = stablehlo.convert %r2 : (tensor<2x3xf32>) -> tensor<2x3xbf16>
        return %c : tensor<2x3xbf16> }""",
}


@pytest.mark.parametrize("name", sorted(PARSE_CASES))
def test_grammar_forms_compile(lib, client, name):
    exe = C.c_void_p()
    rc = lib.mhlo_compile(client, PARSE_CASES[name].encode(), C.byref(exe))
    assert rc == 0, lib.mhlo_get_last_error()
    lib.mhlo_executable_destroy(exe)
