"""Host-only evidence for the two GPU parity bars that are not plain "2e-2 everywhere".

Both tests evaluate the reference's own composition on the CPU more than once and look at how far
those evaluations are from each other and from the exact value; no GPU code runs here.

* Grouped expert FFN (reference composition: csrc/ops/fused_ops.cpp:185-190 over mm / swiglu /
  mul / sum, every result narrowed to the tensor type): two host evaluations that differ only in the
  fp32 summation order of their GEMMs disagree by more than 2e-2 in about one output in ten
  thousand, by exactly one step of the 16-bit result.  A flat 2e-2 bar is therefore not something
  the reference reproduces against itself; the per-element bar max(2e-2, 1 ulp) is.
* Masked attention (csrc/ops/attention_ops.cpp:101-128): here two host evaluations agree to a few
  1e-3, but both are up to 2.4e-2 away from softmax(q k^T s + mask) v evaluated in fp64, because the
  scores are narrowed to 16 bits three times before the softmax.  A kernel that keeps its scores in
  fp32 cannot meet 2e-2 against the host engine; one that narrows at the same places can, which is
  what the masked flash kernels do and what their GPU test asks of them (1e-2)."""
import math

import torch

import oracle as O
from ffn_bar import assert_ffn_close


def test_two_host_evaluations_of_the_expert_ffn_differ_by_one_step_beyond_2e_2():
    """64 tokens of BASELINE config 5's shape (H 4096, I 14336, top-2, weights 0.02 N(0,1), bf16; two
    experts so that the weights fit in seconds): ATen's GEMM against the oracle's C GEMM."""
    torch.manual_seed(0)
    T, H, E, k, I = 64, 4096, 2, 2, 14336
    dt = torch.bfloat16
    logits, x = torch.randn(T, E).to(dt), torch.randn(T, H).to(dt)
    wg, wu = (0.02 * torch.randn(E, I, H)).to(dt), (0.02 * torch.randn(E, I, H)).to(dt)
    wd = (0.02 * torch.randn(E, H, I)).to(dt)
    r = O.moe_route(logits, k)
    a = O.moe_ffn(x, wg, wu, wd, r[1], r[2], r[3], r[5], k, gemm="aten")
    c = O.moe_ffn(x, wg, wu, wd, r[1], r[2], r[3], r[5], k, gemm="c")
    err = (a.double() - c.double()).abs()
    beyond = float((err > 2e-2).double().mean())
    print(f"outputs {err.numel()}: differing {float((err > 0).double().mean()):.2e}, beyond 2e-2 {beyond:.2e}, "
          f"worst {err.max().item():.4f}, max |out| {a.abs().max().item():.3f}")
    # measured: differing 5.9e-3, beyond 2e-2 8.0e-5, worst 0.0625, max |out| 9.875
    assert beyond > 0, "the two host evaluations agree within 2e-2 everywhere: the flat bar would do"
    assert err.max().item() > 2e-2
    assert_ffn_close(c, a, dt)           # ... and they meet the bar the kernel is held to


def test_host_masked_attention_is_reproducible_but_far_from_the_exact_value():
    """The case the masked flash kernel was worst on ([2,4,4,200,200,128] bf16, key-padding mask)."""
    dtype = torch.bfloat16
    B, H, L, D = 2, 4, 200, 128
    worst_between, worst_exact = 0.0, 0.0
    for seed in range(3):
        torch.manual_seed(seed)
        q, k, v = (torch.randn(B, H, L, D).to(dtype) for _ in range(3))
        keep = torch.rand(B, 1, 1, L) > 0.3
        keep[..., :70] &= torch.rand(B, 1, 1, 1) > 0.5
        keep[..., -1] = True
        scale = O.round_to_dtype(1 / math.sqrt(D), dtype)
        for kind in ("bool", "additive"):
            mask = keep if kind == "bool" else (torch.randn(B, 1, 1, L) * 0.5).masked_fill(~keep, -math.inf).to(dtype)
            a, _ = O.sdpa_math(q, k, v, attn_mask=mask, gemm="aten", scale=scale)
            c, _ = O.sdpa_math(q, k, v, attn_mask=mask, gemm="c", scale=scale)
            sc = (q.double() @ k.double().transpose(-1, -2)) * scale
            sc = sc.masked_fill(~mask, -math.inf) if kind == "bool" else sc + mask.double()
            exact = torch.softmax(sc, -1) @ v.double()
            worst_between = max(worst_between, float((a.double() - c.double()).abs().max()))
            worst_exact = max(worst_exact, float((a.double() - exact).abs().max()))
    print(f"host vs host {worst_between:.4f}; host vs fp64 {worst_exact:.4f}")
    # measured: host vs host 0.0020, host vs fp64 0.0237
    assert worst_between <= 5e-3
    assert worst_exact > 1.5e-2
