"""The memory plan made at compile time, without a GPU (METALHLO_ALLOW_NO_DEVICE=1):
every intermediate has a slot in one arena, slots alive together never overlap, values whose
lifetimes are disjoint share bytes.  The plan is what the reference's StaticMemoryPlanner
computes (Sources/MetalHLOCore/Memory/StaticMemoryPlanner.swift:144-250): lifetime-based
offsets at 256-byte alignment."""
import ctypes as C
import os

import pytest

os.environ["METALHLO_ALLOW_NO_DEVICE"] = "1"

from metalhlo_amd import capi  # noqa: E402
from tests import fusion_modules as fm  # noqa: E402


def chain(n_ops, shape="64x64", et="f32"):
    """x -> tanh -> exp -> tanh ... : every intermediate dies right after the next op."""
    t = f"tensor<{shape}x{et}>"
    lines, prev = [], "%x"
    for i in range(n_ops):
        lines.append(f"    %v{i} = stablehlo.{'tanh' if i % 2 == 0 else 'exponential'} {prev} : {t}")
        prev = f"%v{i}"
    return f"func.func @main(%x: {t}) -> {t} {{\n" + "\n".join(lines) + f"\n    return {prev} : {t}\n}}"


@pytest.fixture(scope="module")
def sess():
    lib = capi.load()
    c = C.c_void_p()
    assert lib.mhlo_client_create(C.byref(c)) == 0

    class S:
        pass
    s = S()
    s.lib, s.client = lib, c
    yield s
    lib.mhlo_client_destroy(c)


def plan_of(sess, text, opt=2):
    cfg = capi.CompileConfig()
    sess.lib.mhlo_compile_config_init(C.byref(cfg))
    cfg.optimization_level = opt
    exe = C.c_void_p()
    assert sess.lib.mhlo_compile_with_config(sess.client, text.encode(), C.byref(cfg), C.byref(exe)) == 0, \
        sess.lib.mhlo_get_last_error()
    p = sess.lib.mhlo_ext_executable_plan(exe)
    out = {k: int(v) for k, v in (kv.split("=") for kv in C.string_at(p).decode().split(","))}
    sess.lib.mhlo_free_string(p)
    sess.lib.mhlo_executable_destroy(exe)
    return out


def test_chain_needs_two_slots_of_arena(sess):
    """Ten 16 KiB intermediates in a chain: at any time only a value and its consumer's result
    are alive, so the arena is two slots however long the chain is; the result is not in it."""
    p = plan_of(sess, chain(11))
    assert p["planned"] == 1 and p["slots"] == 11
    assert p["unshared_bytes"] == 10 * 64 * 64 * 4
    assert p["arena_bytes"] == 2 * 64 * 64 * 4
    assert p["result_bytes"] == 64 * 64 * 4
    assert plan_of(sess, chain(41))["arena_bytes"] == 2 * 64 * 64 * 4


def test_offsets_are_256_byte_aligned_and_small_values_round_up(sess):
    p = plan_of(sess, chain(5, shape="3x5"))        # 60-byte values take 256-byte slots
    assert p["arena_bytes"] == 512 and p["unshared_bytes"] == 4 * 256 and p["result_bytes"] == 256


def test_fan_out_keeps_every_live_value_apart(sess):
    """x feeds four branches that are all summed at the end: the four branch results are alive
    together, so the arena cannot be smaller than four of them."""
    t = "tensor<128x128xf32>"
    text = (f"func.func @main(%x: {t}) -> {t} {{\n"
            f"  %a = stablehlo.tanh %x : {t}\n  %b = stablehlo.exponential %x : {t}\n"
            f"  %c = stablehlo.negate %x : {t}\n  %d = stablehlo.abs %x : {t}\n"
            f"  %ab = stablehlo.add %a, %b : {t}\n  %cd = stablehlo.add %c, %d : {t}\n"
            f"  %r = stablehlo.add %ab, %cd : {t}\n  return %r : {t}\n}}")
    p = plan_of(sess, text)
    one = 128 * 128 * 4
    assert p["slots"] == 7 and p["unshared_bytes"] == 6 * one
    assert 4 * one <= p["arena_bytes"] <= 5 * one


def test_temporaries_inside_operations_are_planned(sess):
    """A dot_general whose operands need a transposing copy allocates it inside the op."""
    text = ("func.func @main(%l: tensor<4x3x2xf32>, %r: tensor<5x2x3xf32>) -> tensor<3x4x5xf32> {\n"
            "  %0 = stablehlo.dot_general %l, %r, batching_dims = [1] x [2], contracting_dims = [2] x [1] : "
            "(tensor<4x3x2xf32>, tensor<5x2x3xf32>) -> tensor<3x4x5xf32>\n  return %0 : tensor<3x4x5xf32>\n}")
    p = plan_of(sess, text)
    assert p["planned"] == 1 and p["slots"] == 3 and p["arena_bytes"] == 512      # two copies alive together


def test_unfused_layer_norm_shares_bytes(sess):
    """The decomposed LayerNorm at optimisation level 0 (no pattern recognition) has many short-lived
    intermediates: the arena is clearly smaller than one allocation per value; fused, it has none."""
    p0 = plan_of(sess, fm.LAYER_NORM, opt=0)
    assert p0["planned"] == 1 and p0["slots"] > 5
    assert p0["arena_bytes"] < p0["unshared_bytes"]
    p2 = plan_of(sess, fm.LAYER_NORM, opt=2)
    assert p2["slots"] == 1 and p2["arena_bytes"] == 0


@pytest.mark.parametrize("placement", ["recent", "packed"])
def test_both_placements_keep_live_slots_apart(sess, placement, monkeypatch):
    """Slots are placed where a block of their size was released last (bytes still in the caches)
    unless that takes over a quarter more than packing them at the lowest free address;
    METALHLO_ARENA_PLACEMENT=packed keeps the packed plan.  Either way no two slots alive at the
    same time share a byte, on programs with many sizes and lifetimes."""
    from metalhlo_amd import programs
    monkeypatch.setenv("METALHLO_ARENA_PLACEMENT", placement)
    sizes = {}
    for name, text, opt in [("block", fm.transformer_block(), 2), ("block_as_written", fm.transformer_block(), 0),
                            ("gpt2", programs.gpt2_program(2, 64, 3, 4, 64, 1024, 1000, 128, "bf16"), 2),
                            ("attention", fm.attention(with_mask=True), 0)]:
        p = plan_of(sess, text, opt)
        assert p["planned"] == 1 and p["overlaps"] == 0, name
        assert p["arena_bytes"] <= p["unshared_bytes"]
        sizes[name] = p["arena_bytes"]
    monkeypatch.setenv("METALHLO_ARENA_PLACEMENT", "packed")
    for name, text, opt in [("block", fm.transformer_block(), 2), ("gpt2", programs.gpt2_program(2, 64, 3, 4, 64, 1024, 1000, 128, "bf16"), 2)]:
        assert sizes[name] <= plan_of(sess, text, opt)["arena_bytes"] * 5 // 4
