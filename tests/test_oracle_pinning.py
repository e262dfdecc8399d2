"""Pins the CPU oracle (oracle/paras_oracle.c + oracle/oracle.py) before anything
is measured against it.

Three independent anchors, as the reference's own tests use them:
  1. the reference's own CPU flavor, compiled from its sources into
     oracle/_ref (bit-for-bit, in a child process because it claims the
     PrivateUse1 device);
  2. closed forms and torch-CPU library routines at the reference's test
     tolerance (tests/common.py:7-8 -> 1e-4), on the shapes its tests use
     (tests/test_fused_ops.py:8-70, tests/test_attention_norm_ops.py:35-165,
     tests/test_pointwise_ops.py:224-267,369-413,
     tests/test_matmul_sort_creation_ops.py:133-139);
  3. brute force / invariants that a dropped term, a wrong sign or a transposed
     operand would break.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle as O
import ref_engine as R
from conftest import assert_bit_exact

ATOL = RTOL = 1e-4  # reference tests/common.py:7-8
DTYPES = [torch.float32, torch.bfloat16, torch.float16, torch.float64]

needs_ref = pytest.mark.skipif(not R.available(), reason="oracle/_ref not built (reference sources absent)")


def close(a, b):
    assert a.dtype == b.dtype and a.shape == b.shape
    assert torch.allclose(a, b, atol=ATOL, rtol=RTOL, equal_nan=True), (a - b).abs().max()


# --------------------------------------------------------------------------- 1
@needs_ref
@pytest.mark.parametrize("dtype", DTYPES)
def test_oracle_equals_reference_engine_bitwise(dtype):
    """Every oracle function against the reference's compiled host engine."""
    g = torch.Generator().manual_seed(1)
    rn = lambda *s: torch.randn(*s, generator=g)
    x, w, go = rn(37, 200).to(dtype), (1 + 0.02 * rn(200)).to(dtype), rn(37, 200).to(dtype)
    gate, up, gs = (3 * rn(33, 70)).to(dtype), rn(33, 70).to(dtype), rn(33, 70).to(dtype)
    q, k, v = rn(2, 4, 8, 16).to(dtype), rn(2, 4, 8, 16).to(dtype), rn(2, 4, 8, 16).to(dtype)
    kg, vg = rn(2, 2, 8, 16).to(dtype), rn(2, 2, 8, 16).to(dtype)
    mask = torch.rand(2, 4, 8, 8, generator=g) > 0.3
    bias = (0.1 * rn(2, 4, 8, 8)).to(dtype)
    logits = rn(50, 8).to(dtype)
    logits[3] = logits[3, 0]  # a fully tied row
    x3 = rn(3, 4, 5).to(dtype)

    jobs = {
        "rms_norm": ((x, w, 1e-6), {}),
        "swiglu": ((gate, up), {}),
        "swiglu_backward": ((gs, gate, up), {}),
        "rotate_half": ((x,), {}),
        "rms_norm_composed": ((x, [200], w, 1e-5), {}),
        "swiglu_composed": ((gate, up), {}),
        "softmax_last": ((rn(9, 77).to(dtype),), {}),
        "topk_last": ((logits, 3), {}),
        "moe_route": ((logits, 2), {}),
    }
    out, rstd = O.rms_norm(x, w, 1e-6)
    variants = [dict(), dict(is_causal=True), dict(attn_mask=mask), dict(attn_mask=bias), dict(scale=1 / math.sqrt(32))]
    batch = [(name, args, kw) for name, (args, kw) in jobs.items()]
    batch += [("rms_norm_backward", (go, x, w, rstd), {}), ("rotate_half", (x, True), {}),
              ("rms_norm_composed", (x3, [4, 5]), {})]
    batch += [("sdpa_math", (q, k, v), kw) for kw in variants]
    batch += [("sdpa_math", (q, kg, vg), dict(enable_gqa=True))]
    # the glue primitives: add / sub (with alpha) / mul / div of tensors (one broadcast) and of a
    # tensor with a number, and the row gather of the MoE permutation
    a2, b2, row = rn(6, 70).to(dtype), (rn(6, 70) + 2.5).to(dtype), rn(70).to(dtype)
    idx = torch.tensor([5, 0, 0, 3, 2, 5, 1])
    glue = [("binary", (O.OP_ADD, a2, b2, 1.0), {}), ("binary", (O.OP_ADD, a2, b2, -0.75), {}), ("binary", (O.OP_SUB, a2, b2, 1.0), {}),
            ("binary", (O.OP_SUB, a2, row, 2.5), {}), ("binary", (O.OP_MUL, a2, row), {}), ("binary", (O.OP_DIV, a2, b2), {}),
            ("binary_scalar", (O.OP_ADD, a2, 0.3, 1.0), {}), ("binary_scalar", (O.OP_SUB, a2, 0.3, 2.0), {}),
            ("binary_scalar", (O.OP_MUL, a2, 1 / math.sqrt(128)), {}), ("binary_scalar", (O.OP_DIV, a2, 3.0), {}),
            ("index_select_rows", (a2, idx), {})]
    n_glue0 = len(batch)
    batch += glue
    results = R.run_batch(batch)          # one child process: the engine owns PrivateUse1

    def same(got, want, what):
        if not isinstance(want, (tuple, list)):
            want, got = (want,), (got,)
        for i, (a, b) in enumerate(zip(got, want)):
            assert_bit_exact(a, b, f"{what}[{i}] {dtype}")

    n = len(jobs)
    for (name, (args, kw)), want in zip(jobs.items(), results[:n]):
        same(getattr(O, name)(*args, **kw), want, name)
    same(O.rms_norm_backward(go, x, w, rstd), results[n], "rms_norm_backward")
    same(O.rotate_half(x, True), results[n + 1], "rotate_half_backward")
    same(O.rms_norm_composed(x3, [4, 5]), results[n + 2], "rms multi-dim")

    # SDPA: with the GEMM the reference itself bounces to (ATen-CPU) every
    # variant is bit-identical; the C double-accumulate GEMM is compared at the
    # dtype's own resolution.
    for kw, want in zip(variants, results[n + 3:n + 3 + len(variants)]):
        same(O.sdpa_math(q, k, v, gemm="aten", **kw), want, f"sdpa {sorted(kw)}")
        alt = O.sdpa_math(q, k, v, gemm="c", **kw)
        tol = {torch.float32: 2e-6, torch.float64: 1e-14, torch.bfloat16: 1.6e-2, torch.float16: 2e-3}[dtype]
        assert (alt[0].double() - want[0].double()).abs().max() <= tol
    same(O.sdpa_math(q, kg, vg, enable_gqa=True, gemm="aten"), results[n_glue0 - 1], "sdpa gqa")
    for (name, args, kw), want in zip(glue, results[n_glue0:]):
        same(getattr(O, name)(*args, **kw), want, f"{name} op {args[0] if name != 'index_select_rows' else ''}")


@needs_ref
def test_oracle_moe_ffn_equals_reference_composition():
    """The canonical MoE composition, run primitive by primitive on the
    reference engine, against the oracle's restatement (same ATen GEMM)."""
    g = torch.Generator().manual_seed(2)
    T, E, k, H, I = 40, 4, 2, 32, 48
    dt = torch.bfloat16
    x = torch.randn(T, H, generator=g).to(dt)
    logits = torch.randn(T, E, generator=g).to(dt)
    wg, wu = (0.2 * torch.randn(E, I, H, generator=g)).to(dt), (0.2 * torch.randn(E, I, H, generator=g)).to(dt)
    wd = (0.2 * torch.randn(E, H, I, generator=g)).to(dt)
    topi, topw, order, inv, counts, offsets = O.moe_route(logits, k)
    want = R.run("moe_ffn", x, wg, wu, wd, topw, order, inv, offsets, k)
    got = O.moe_ffn(x, wg, wu, wd, topw, order, inv, offsets, k, gemm="aten")
    assert_bit_exact(got, want, "moe_ffn")


# --------------------------------------------------------------------------- 2
def test_rms_norm_closed_form():
    x, w = torch.randn(4, 8), torch.randn(8)
    ref = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w  # tests/test_fused_ops.py:8-17
    out, rstd = O.rms_norm(x, w, 1e-6)
    close(out, ref)
    close(rstd, torch.rsqrt(x.pow(2).mean(-1) + 1e-6))


def test_rms_norm_backward_matches_autograd():
    x = torch.randn(4, 8, requires_grad=True)
    w = torch.randn(8, requires_grad=True)
    (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w).sum().backward()
    out, rstd = O.rms_norm(x.detach(), w.detach(), 1e-6)
    gx, gw = O.rms_norm_backward(torch.ones(4, 8), x.detach(), w.detach(), rstd)
    close(gx, x.grad)
    close(gw, w.grad)


def test_swiglu_closed_form_and_backward():
    gate = torch.randn(4, 8, requires_grad=True)
    up = torch.randn(4, 8, requires_grad=True)
    ref = F.silu(gate) * up
    ref.sum().backward()
    close(O.swiglu(gate.detach(), up.detach()), ref.detach())
    gg, gu = O.swiglu_backward(torch.ones(4, 8), gate.detach(), up.detach())
    close(gg, gate.grad)
    close(gu, up.grad)
    # the composed op has its operands the other way round: x * silu(gate)
    close(O.swiglu_composed(up.detach(), gate.detach()), (up * F.silu(gate)).detach())


def test_rotate_half_closed_form():
    x = torch.randn(4, 8)
    x1, x2 = x.chunk(2, dim=-1)
    assert torch.equal(O.rotate_half(x), torch.cat((-x2, x1), dim=-1))
    assert torch.equal(O.rotate_half(x, backward=True), torch.cat((x2, -x1), dim=-1))


def test_aten_rms_norm_variants():
    x = torch.randn(4, 6, 32)
    close(O.rms_norm_composed(x, [32]), torch.ops.aten.rms_norm(x, [32], None, 1e-6))
    w = torch.randn(32)
    close(O.rms_norm_composed(x, [32], w, 1e-5), torch.ops.aten.rms_norm(x, [32], w, 1e-5))
    x3 = torch.randn(3, 4, 5)
    close(O.rms_norm_composed(x3, [4, 5]), torch.ops.aten.rms_norm(x3, [4, 5], None, 1e-6))
    with pytest.raises(AssertionError):
        O.rms_norm_composed(x, [32], torch.randn(16))


@pytest.mark.parametrize("kw", [dict(), dict(is_causal=True), dict(scale=1 / math.sqrt(32))])
def test_sdpa_against_torch_cpu(kw):
    q, k, v = torch.randn(2, 4, 8, 16), torch.randn(2, 4, 8, 16), torch.randn(2, 4, 8, 16)
    close(O.sdpa_math(q, k, v, **kw)[0], F.scaled_dot_product_attention(q, k, v, **kw))


def test_sdpa_causal_is_top_left_aligned():
    """Lq != Lk: query i sees keys 0..i (tests/test_attention_norm_ops.py:57-62)."""
    q, k, v = torch.randn(2, 4, 4, 16), torch.randn(2, 4, 8, 16), torch.randn(2, 4, 8, 16)
    out, attn = O.sdpa_math(q, k, v, is_causal=True)
    close(out, F.scaled_dot_product_attention(q, k, v, is_causal=True))
    assert torch.equal(attn[..., 0, 1:], torch.zeros(2, 4, 7))     # row 0 sees key 0 only
    close(out[..., 0, :], v[..., 0, :])


def test_sdpa_masks_and_gqa():
    q, k, v = torch.randn(2, 4, 8, 16), torch.randn(2, 4, 8, 16), torch.randn(2, 4, 8, 16)
    mask = torch.rand(2, 4, 8, 8) > 0.3
    close(O.sdpa_math(q, k, v, attn_mask=mask)[0], F.scaled_dot_product_attention(q, k, v, attn_mask=mask))
    bias = torch.randn(2, 4, 8, 8) * 0.1
    close(O.sdpa_math(q, k, v, attn_mask=bias)[0], F.scaled_dot_product_attention(q, k, v, attn_mask=bias))
    kg, vg = torch.randn(2, 2, 8, 16), torch.randn(2, 2, 8, 16)
    want = F.scaled_dot_product_attention(q, kg.repeat_interleave(2, 1), vg.repeat_interleave(2, 1))
    close(O.sdpa_math(q, kg, vg, enable_gqa=True)[0], want)


def test_sdpa_invariants():
    q, k, v = torch.randn(1, 2, 16, 8), torch.randn(1, 2, 16, 8), torch.randn(1, 2, 16, 8)
    out, attn = O.sdpa_math(q, k, v, is_causal=True)
    close(attn.sum(-1), torch.ones(1, 2, 16))
    # q = 0 -> uniform weights -> causal prefix mean of v
    out0, _ = O.sdpa_math(torch.zeros_like(q), k, v, is_causal=True)
    close(out0, torch.cumsum(v, 2) / torch.arange(1, 17).view(1, 1, 16, 1))


def test_softmax_and_topk_against_torch():
    x = torch.randn(5, 33)
    close(O.softmax_last(x), torch.softmax(x, -1))
    assert O.softmax_last(x.bfloat16(), torch.float32).dtype == torch.float32
    vals, idx = O.topk_last(x, 4)
    tv, ti = torch.topk(x, 4, dim=-1)
    assert torch.equal(vals, tv) and torch.equal(idx, ti)
    # ties: lower index first, output sorted (tests/test_pointwise_ops.py:405-413 literal)
    t = torch.tensor([[5., 3., 5., 5., 1., 3.]])
    vals, idx = O.topk_last(t, 4)
    assert vals.tolist() == [[5., 5., 5., 3.]] and idx.tolist() == [[0, 2, 3, 1]]
    vals, idx = O.topk_last(t, 2, largest=False)
    assert vals.tolist() == [[1., 3.]] and idx.tolist() == [[4, 1]]


def test_topk_brute_force_with_ties():
    x = torch.randint(0, 4, (200, 8)).float()
    vals, idx = O.topk_last(x, 3)
    for r in range(200):
        want = sorted(range(8), key=lambda j: (-x[r, j].item(), j))[:3]
        assert idx[r].tolist() == want


def test_stable_argsort_and_routing_invariants():
    t = torch.tensor([3, 1, 2, 1, 3])  # tests/test_pointwise_ops.py:454-459 literal
    assert O.argsort_stable(t).tolist() == [1, 3, 2, 0, 4]
    keys = torch.randint(0, 8, (1000,))
    assert torch.equal(O.argsort_stable(keys), torch.argsort(keys, stable=True))
    logits = torch.randn(500, 8).bfloat16()
    topi, topw, order, inv, counts, offsets = O.moe_route(logits, 2)
    flat = topi.reshape(-1)
    assert sorted(order.tolist()) == list(range(1000))            # a permutation
    assert bool((flat[order][1:] >= flat[order][:-1]).all())       # expert-major
    for e in range(8):                                             # stable inside an expert
        seg = order[offsets[e]:offsets[e + 1]]
        assert bool((seg[1:] > seg[:-1]).all())
    assert counts.sum().item() == 1000 and offsets[-1].item() == 1000
    assert torch.equal(inv[order], torch.arange(1000))
    close(topw.sum(-1), torch.ones(500))
    full = torch.softmax(logits.float(), -1).gather(1, topi)       # softmax-then-renormalise is the same gate
    close(topw, full / full.sum(-1, keepdim=True))


def test_moe_ffn_against_dense_formula():
    T, E, k, H, I = 24, 4, 2, 16, 32
    x, logits = torch.randn(T, H), torch.randn(T, E)
    wg, wu, wd = torch.randn(E, I, H) * 0.3, torch.randn(E, I, H) * 0.3, torch.randn(E, H, I) * 0.3
    topi, topw, order, inv, counts, offsets = O.moe_route(logits, k)
    got = O.moe_ffn(x, wg, wu, wd, topw, order, inv, offsets, k)
    want = torch.zeros(T, H)
    for t in range(T):
        for s in range(k):
            e = topi[t, s]
            want[t] += topw[t, s] * ((F.silu(x[t] @ wg[e].T) * (x[t] @ wu[e].T)) @ wd[e].T)
    close(got, want)


def test_dtype_narrowing_is_double_float_then_16bit():
    # 1 + 2^-8 + 2^-30: straight double->bf16 rounds up, double->float->bf16 ties to even (down)
    v = 1.0 + 2.0 ** -8 + 2.0 ** -30
    assert O.round_to_dtype(v, torch.bfloat16) == 1.0
    assert O.round_to_dtype(1.0 + 2.0 ** -8 + 2.0 ** -20, torch.bfloat16) == 1.0 + 2.0 ** -7
    x = torch.randn(100000, dtype=torch.float64) * torch.logspace(-9, 5, 100000, dtype=torch.float64)
    for dt in (torch.float16, torch.bfloat16):
        got = torch.tensor([O.round_to_dtype(float(t), dt) for t in x[:5000]], dtype=torch.float64)
        assert torch.equal(got, x[:5000].float().to(dt).double())


def test_empty_inputs():
    out, rstd = O.rms_norm(torch.empty(0, 8), torch.ones(8), 1e-6)
    assert out.shape == (0, 8) and rstd.shape == (0,)
    assert O.swiglu(torch.empty(0, 4), torch.empty(0, 4)).shape == (0, 4)
