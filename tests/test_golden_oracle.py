"""The CPU oracle against the committed golden vectors (outputs of the
reference's host engine).  Runs anywhere, with or without oracle/_ref."""
import math

import pytest
import torch

import oracle as O
from conftest import assert_bit_exact
from golden_util import DTYPE_TAGS, case


@pytest.mark.parametrize("tag", DTYPE_TAGS)
def test_fused_ops(tag):
    c = case(f"rms_norm_{tag}")
    out, rstd = O.rms_norm(c["x"], c["w"], 1e-6)
    assert_bit_exact(out, c["out"], "rms_norm")
    assert_bit_exact(rstd, c["rstd"], "rstd")
    gx, gw = O.rms_norm_backward(c["go"], c["x"], c["w"], c["rstd"])
    assert_bit_exact(gx, c["gx"], "rms_norm grad_input")
    assert_bit_exact(gw, c["gw"], "rms_norm grad_weight")
    c = case(f"swiglu_{tag}")
    assert_bit_exact(O.swiglu(c["gate"], c["up"]), c["out"], "swiglu")
    gg, gu = O.swiglu_backward(c["go"], c["gate"], c["up"])
    assert_bit_exact(gg, c["ggate"], "swiglu grad_gate")
    assert_bit_exact(gu, c["gup"], "swiglu grad_up")
    c = case(f"rotate_half_{tag}")
    assert_bit_exact(O.rotate_half(c["x"]), c["out"], "rotate_half")
    assert_bit_exact(O.rotate_half(c["x"], True), c["bwd"], "rotate_half_backward")


@pytest.mark.parametrize("tag", DTYPE_TAGS)
def test_composed_ops(tag):
    c = case(f"rms_composed_{tag}")
    assert_bit_exact(O.rms_norm_composed(c["x"], [264], c["w"], 1e-5), c["out"], "aten::rms_norm")
    assert_bit_exact(O.rms_norm_composed(c["x"], [264]), c["out_now"], "aten::rms_norm no weight")
    c = case(f"swiglu_composed_{tag}")
    assert_bit_exact(O.swiglu_composed(c["x"], c["gate"]), c["out"], "torch_paras::swiglu")


@pytest.mark.parametrize("tag", DTYPE_TAGS)
def test_sdpa(tag):
    c = case(f"sdpa_{tag}")
    q, k, v = c["q"], c["k"], c["v"]
    variants = {"plain": {}, "causal": dict(is_causal=True), "bool": dict(attn_mask=c["mask"].bool()),
                "bias": dict(attn_mask=c["bias"]), "scale": dict(scale=1 / math.sqrt(32))}
    for name, kw in variants.items():
        out, attn = O.sdpa_math(q, k, v, gemm="aten", **kw)
        assert_bit_exact(out, c[f"out_{name}"], f"sdpa {name} out")
        assert_bit_exact(attn, c[f"attn_{name}"], f"sdpa {name} attn")
    out, attn = O.sdpa_math(q, c["kg"], c["vg"], enable_gqa=True, gemm="aten")
    assert_bit_exact(out, c["out_gqa"], "sdpa gqa out")


@pytest.mark.parametrize("tag", ("bf16", "f16"))
def test_sdpa_head128_and_decode(tag):
    c = case(f"sdpa_d128_{tag}")
    assert_bit_exact(O.sdpa_math(c["q"], c["k"], c["v"], is_causal=True, enable_gqa=True, gemm="aten")[0],
                     c["out_causal"], "causal gqa d128")
    d = case(f"sdpa_decode_{tag}")
    assert_bit_exact(O.sdpa_math(d["q"], c["k"], c["v"], enable_gqa=True, gemm="aten")[0], d["out"], "decode")


@pytest.mark.parametrize("tag", DTYPE_TAGS)
def test_moe_route(tag):
    c = case(f"moe_route_{tag}")
    got = O.moe_route(c["logits"], 2)
    for name, g in zip(("topi", "topw", "order", "inv", "counts", "offsets"), got):
        assert_bit_exact(g, c[name], f"moe_route {name}")


def test_moe_ffn_and_literals():
    c = case("moe_ffn_bf16")
    got = O.moe_ffn(c["x"], c["wg"], c["wu"], c["wd"], c["topw"], c["order"], c["inv"], c["offsets"], 2, gemm="aten")
    assert_bit_exact(got, c["out"], "moe_ffn")
    t = case("topk_ties_literal")
    vals, idx = O.topk_last(t["x"], 4)
    assert torch.equal(vals, t["vals"]) and torch.equal(idx, t["idx"])
    a = case("argsort_literal")
    assert torch.equal(O.argsort_stable(a["x"]), a["out"])


@pytest.mark.parametrize("tag", DTYPE_TAGS)
def test_glue_primitives(tag):
    """add / sub (alpha) / mul / div of tensors and of a tensor with a number, and the row gather."""
    c = case(f"glue_{tag}")
    a, b, row = c["a"], c["b"], c["row"]
    assert_bit_exact(O.binary(O.OP_ADD, a, b, 1.0), c["add"], "add")
    assert_bit_exact(O.binary(O.OP_ADD, a, b, -0.75), c["add_alpha"], "add alpha")
    assert_bit_exact(O.binary(O.OP_SUB, a, b, 1.0), c["sub"], "sub")
    assert_bit_exact(O.binary(O.OP_SUB, a, row, 2.5), c["sub_row_alpha"], "sub broadcast alpha")
    assert_bit_exact(O.binary(O.OP_MUL, a, row), c["mul_row"], "mul broadcast")
    assert_bit_exact(O.binary(O.OP_DIV, a, b), c["div"], "div")
    assert_bit_exact(O.binary_scalar(O.OP_ADD, a, 0.3, 1.0), c["add_s"], "add number")
    assert_bit_exact(O.binary_scalar(O.OP_SUB, a, 0.3, 2.0), c["sub_s_alpha"], "sub number alpha")
    assert_bit_exact(O.binary_scalar(O.OP_MUL, a, 1 / math.sqrt(128)), c["mul_s"], "mul number")
    assert_bit_exact(O.binary_scalar(O.OP_DIV, a, 3.0), c["div_s"], "div number")
    assert_bit_exact(O.index_select_rows(a, c["idx"]), c["rows"], "index_select rows")
