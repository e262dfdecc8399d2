"""The drop-in surface: `import torch_paras`, the `paras` device, the aten /
paras:: / torch_paras:: ops, driven the way the reference's own tests drive
them (tests/test_attention_norm_ops.py, tests/test_fused_ops.py, copy tests of
tests/test_attention_norm_ops.py:172-216) -- device result against torch-CPU at
the reference's tolerance, plus the oracle for the 16-bit dtypes."""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle as O
from conftest import assert_bit_exact

pytestmark = pytest.mark.gpu
ATOL = RTOL = 1e-4  # reference tests/common.py:7-8


@pytest.fixture(scope="module")
def device():
    import torch_paras
    assert torch_paras.is_available() and torch_paras.backend_name() == "paras-hip"
    return "paras:0"


def assert_close(actual, expected, msg=""):
    actual, expected = actual.cpu(), expected.cpu()
    assert actual.dtype == expected.dtype, f"{msg}: dtype {actual.dtype} vs {expected.dtype}"
    assert actual.shape == expected.shape, f"{msg}: shape {tuple(actual.shape)} vs {tuple(expected.shape)}"
    if actual.dtype.is_floating_point:
        assert torch.allclose(actual, expected, atol=ATOL, rtol=RTOL, equal_nan=True), msg
    else:
        assert torch.equal(actual, expected), msg


def _qkv(device, B=2, H=4, Lq=8, Lk=8, E=16, dtype=torch.float32):
    q, k, v = torch.randn(B, H, Lq, E, dtype=dtype), torch.randn(B, H, Lk, E, dtype=dtype), torch.randn(B, H, Lk, E, dtype=dtype)
    return q, k, v, q.to(device), k.to(device), v.to(device)


# ---- module surface -----------------------------------------------------------
def test_module_surface(device):
    import torch_paras
    assert torch_paras.device_count() >= 1 and torch.paras.is_available()
    assert isinstance(torch_paras.device_name(0), str) and torch_paras.is_gpu_device(0)
    assert torch_paras.get_amp_supported_dtype() == [torch.float16, torch.float32]
    assert torch.paras._is_in_bad_fork() is False
    x = torch.randn(1000, 1000).to(device)
    assert x.is_paras and x.device == torch.device("paras", 0)
    assert torch_paras.memory_allocated(0) >= 4_000_000
    del x
    torch_paras.synchronize()
    torch_paras.empty_cache()
    assert torch_paras.memory_cached(0) == 0
    torch_paras.manual_seed(0)
    with pytest.raises(RuntimeError):
        torch.randn(2).to("paras:7")


# ---- scaled dot-product attention (reference tests/test_attention_norm_ops.py:35-108)
def test_sdpa_basic(device):
    q, k, v, dq, dk, dv = _qkv(device)
    assert_close(F.scaled_dot_product_attention(dq, dk, dv), F.scaled_dot_product_attention(q, k, v), "sdpa_basic")


def test_sdpa_explicit_scale(device):
    q, k, v, dq, dk, dv = _qkv(device, E=16)
    s = 1.0 / math.sqrt(32)
    assert_close(F.scaled_dot_product_attention(dq, dk, dv, scale=s), F.scaled_dot_product_attention(q, k, v, scale=s), "scale")


def test_sdpa_causal(device):
    q, k, v, dq, dk, dv = _qkv(device)
    assert_close(F.scaled_dot_product_attention(dq, dk, dv, is_causal=True),
                 F.scaled_dot_product_attention(q, k, v, is_causal=True), "causal")


def test_sdpa_fp32_at_a_size_that_runs_composed(device):
    """fp32 (the reference's default dtype) at a thousand tokens: batched products and one row kernel
    inside the library, workspace from the device pool; also through the math op with its weights."""
    q, k, v, dq, dk, dv = _qkv(device, B=1, H=8, Lq=1024, Lk=1024, E=64)
    assert_close(F.scaled_dot_product_attention(dq, dk, dv, is_causal=True),
                 F.scaled_dot_product_attention(q, k, v, is_causal=True), "fp32 causal, 1024 tokens")
    out, attn = torch.ops.aten._scaled_dot_product_attention_math(dq, dk, dv, is_causal=True)
    want, wattn = torch.ops.aten._scaled_dot_product_attention_math(q, k, v, is_causal=True)
    assert_close(out, want, "math op out")
    assert_close(attn, wattn, "math op weights")
    x, w = torch.randn(1024, 768), torch.randn(1536, 768) / 28.0          # an fp32 projection on the matrix cores
    assert_close(F.linear(x.to(device), w.to(device)), F.linear(x, w), "fp32 linear")


def test_sdpa_causal_unequal_lengths(device):
    q, k, v, dq, dk, dv = _qkv(device, Lq=4, Lk=8)
    assert_close(F.scaled_dot_product_attention(dq, dk, dv, is_causal=True),
                 F.scaled_dot_product_attention(q, k, v, is_causal=True), "causal Lq != Lk")


def test_sdpa_bool_mask(device):
    q, k, v, dq, dk, dv = _qkv(device)
    mask = torch.rand(2, 4, 8, 8) > 0.3
    assert_close(F.scaled_dot_product_attention(dq, dk, dv, attn_mask=mask.to(device)),
                 F.scaled_dot_product_attention(q, k, v, attn_mask=mask), "bool mask")
    m2 = torch.rand(8, 8) > 0.3            # broadcast over batch and heads
    m2[:, 0] = True
    assert_close(F.scaled_dot_product_attention(dq, dk, dv, attn_mask=m2.to(device)),
                 F.scaled_dot_product_attention(q, k, v, attn_mask=m2), "broadcast bool mask")


def test_sdpa_bf16_key_padding_mask_and_bias(device):
    """The shapes a padded batch produces: bf16, a [B, 1, 1, Lk] bool mask, then an fp32 additive
    bias (converted to the tensors' dtype, attention_ops.cpp:122-125).  Checked against torch's
    own CPU result on the same bf16 inputs evaluated in fp32."""
    B, H, L, D = 2, 4, 160, 64
    q, k, v = (torch.randn(B, H, L, D).bfloat16() for _ in range(3))
    lengths = torch.tensor([160, 97])
    pad = torch.arange(L)[None, :] < lengths[:, None]                 # [B, L]
    mask = pad[:, None, None, :]
    got = F.scaled_dot_product_attention(q.to(device), k.to(device), v.to(device), attn_mask=mask.to(device)).cpu()
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)
    assert got.dtype == torch.bfloat16 and float((got.float() - want).abs().max()) <= 2e-2
    bias = torch.randn(1, H, L, L) * 0.5
    got = F.scaled_dot_product_attention(q.to(device), k.to(device), v.to(device), attn_mask=bias.to(device)).cpu()
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=bias.bfloat16().float())
    assert float((got.float() - want).abs().max()) <= 2e-2


@pytest.mark.parametrize("D", [96, 80, 40, 192, 256])
def test_sdpa_16bit_other_head_sizes_run_zero_padded(device, D):
    """Head sizes other than 64 / 128 / 256 go through the MFMA kernels with zero columns appended
    (the default scale stays 1/sqrt(D) of the real size); results as for any other 16-bit call."""
    B, H, L = 2, 3, 150
    q, k, v = (torch.randn(B, H, L, D).half() for _ in range(3))
    got = F.scaled_dot_product_attention(q.to(device), k.to(device), v.to(device), is_causal=True).cpu()
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True)
    assert got.shape == (B, H, L, D) and got.dtype == torch.float16 and got.is_contiguous()
    assert float((got.float() - want).abs().max()) <= 2e-2
    mask = torch.rand(B, 1, L, L) > 0.4
    mask[..., 0] = True
    got = F.scaled_dot_product_attention(q.to(device), k.to(device), v.to(device), attn_mask=mask.to(device), scale=0.2).cpu()
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask, scale=0.2)
    assert float((got.float() - want).abs().max()) <= 2e-2


def test_sdpa_additive_mask(device):
    q, k, v, dq, dk, dv = _qkv(device)
    bias = torch.randn(2, 4, 8, 8) * 0.1
    assert_close(F.scaled_dot_product_attention(dq, dk, dv, attn_mask=bias.to(device)),
                 F.scaled_dot_product_attention(q, k, v, attn_mask=bias), "additive mask")


def test_sdpa_gqa(device):
    B, Lq, Lk, E = 2, 8, 8, 16
    q, k, v = torch.randn(B, 4, Lq, E), torch.randn(B, 2, Lk, E), torch.randn(B, 2, Lk, E)
    ref, ref_w = torch.ops.aten._scaled_dot_product_attention_math(q, k, v, None, 0.0, False, None, scale=None, enable_gqa=True)
    out, w = torch.ops.aten._scaled_dot_product_attention_math(q.to(device), k.to(device), v.to(device), None, 0.0, False,
                                                               None, scale=None, enable_gqa=True)
    assert_close(out, ref, "sdpa_gqa")
    assert_close(w, ref_w, "sdpa_gqa weights")
    assert_close(F.scaled_dot_product_attention(q.to(device), k.to(device), v.to(device), enable_gqa=True), ref, "F.sdpa gqa")


def test_sdpa_mismatched_gqa_heads_raises(device):
    q, k, v = torch.randn(1, 5, 4, 8).to(device), torch.randn(1, 2, 4, 8).to(device), torch.randn(1, 2, 4, 8).to(device)
    with pytest.raises(RuntimeError):
        torch.ops.aten._scaled_dot_product_attention_math(q, k, v, None, 0.0, False, None, scale=None, enable_gqa=True)
    with pytest.raises(RuntimeError):
        torch.ops.aten._scaled_dot_product_attention_math(q, k, v, torch.ones(4, 4, dtype=torch.bool).to(device), 0.0, True, None)


def test_sdpa_math_op_returns_host_engine_weights(device):
    """bf16: the math op's weights equal the host engine's bit for bit."""
    q, k, v = (torch.randn(2, 4, 8, 16).bfloat16() for _ in range(3))
    out, w = torch.ops.aten._scaled_dot_product_attention_math(q.to(device), k.to(device), v.to(device), None, 0.0, True, None)
    want, want_w = O.sdpa_math(q, k, v, is_causal=True, gemm="aten")
    assert_bit_exact(w.cpu(), want_w, "weights")
    assert (out.cpu().float() - want.float()).abs().max().item() <= 2 ** -7


def test_sdpa_bf16_takes_the_flash_and_decode_kernels(device):
    q, k, v = (torch.randn(2, 8, 256, 128).bfloat16() for _ in range(3))
    out = F.scaled_dot_product_attention(q.to(device), k.to(device), v.to(device), is_causal=True)
    want, _ = O.sdpa_math(q, k, v, is_causal=True, gemm="aten")
    assert out.dtype == torch.bfloat16 and (out.cpu().float() - want.float()).abs().max().item() <= 2e-2
    q1, k1, v1 = torch.randn(2, 8, 1, 128).bfloat16(), torch.randn(2, 2, 777, 128).bfloat16(), torch.randn(2, 2, 777, 128).bfloat16()
    out = F.scaled_dot_product_attention(q1.to(device), k1.to(device), v1.to(device), enable_gqa=True)
    want, _ = O.sdpa_math(q1, k1, v1, enable_gqa=True, gemm="aten")
    assert (out.cpu().float() - want.float()).abs().max().item() <= 2e-2
    q3 = torch.randn(4, 64, 128).bfloat16()                      # 3-D input
    out = F.scaled_dot_product_attention(q3.to(device), q3.to(device), q3.to(device))
    want, _ = O.sdpa_math(q3, q3, q3, gemm="aten")
    assert out.shape == (4, 64, 128) and (out.cpu().float() - want.float()).abs().max().item() <= 2e-2


# ---- aten::rms_norm / torch_paras::swiglu (reference tests/test_attention_norm_ops.py:115-165)
def test_sdpa_views_at_odd_offsets_still_take_the_mfma_kernels(device):
    """q / k / v that start off a 16-byte boundary, or whose strides are not multiples of 8 elements,
    are copied dense before the call: no general-kernel launch, same values as from fresh tensors."""
    import torch_paras
    B, H, L, D = 1, 4, 256, 128
    q, k, v = (torch.randn(B, H, L, D).bfloat16() for _ in range(3))
    want = F.scaled_dot_product_attention(q.to(device), k.to(device), v.to(device), is_causal=True).cpu()

    def shifted(t, extra_row=0):
        buf = torch.empty(B * H * L * (D + extra_row) + 1, dtype=t.dtype).to(device)
        view = buf[1:].view(B, H, L, D + extra_row)[..., :D]
        view.copy_(t.to(device))
        return view
    got = F.scaled_dot_product_attention(shifted(q), shifted(k), shifted(v), is_causal=True).cpu()
    assert_bit_exact(got, want, "sdpa from views one element off a boundary")
    got = F.scaled_dot_product_attention(shifted(q, 3), shifted(k, 3), shifted(v, 3), is_causal=True).cpu()
    assert_bit_exact(got, want, "sdpa from views with odd row strides")


def test_rms_norm_no_weight(device):
    x = torch.randn(4, 6, 32)
    assert_close(torch.ops.aten.rms_norm(x.to(device), [32], None, None), torch.ops.aten.rms_norm(x, [32], None, 1e-6), "no weight")


def test_rms_norm_with_weight(device):
    x, w = torch.randn(4, 6, 32), torch.randn(32)
    assert_close(torch.ops.aten.rms_norm(x.to(device), [32], w.to(device), 1e-5), torch.ops.aten.rms_norm(x, [32], w, 1e-5), "weight")


def test_rms_norm_multi_dim_normalized_shape(device):
    x = torch.randn(3, 4, 5)
    assert_close(torch.ops.aten.rms_norm(x.to(device), [4, 5], None, None), torch.ops.aten.rms_norm(x, [4, 5], None, 1e-6), "multi-dim")


def test_rms_norm_shape_mismatch_raises(device):
    with pytest.raises(RuntimeError):
        torch.ops.aten.rms_norm(torch.randn(4, 6, 32).to(device), [32], torch.randn(16).to(device), None)


def test_composed_ops_narrow_like_the_host_engine(device):
    for dt in (torch.bfloat16, torch.float16, torch.float32):
        x, w = torch.randn(37, 200).to(dt), (1 + 0.02 * torch.randn(200)).to(dt)
        got = torch.ops.aten.rms_norm(x.to(device), [200], w.to(device), 1e-5)
        assert_bit_exact(got.cpu(), O.rms_norm_composed(x, [200], w, 1e-5), f"aten::rms_norm {dt}")
        g = (3 * torch.randn(33, 70)).to(dt)
        u = torch.randn(33, 70).to(dt)
        got = torch.ops.torch_paras.swiglu(u.to(device), g.to(device))
        assert_bit_exact(got.cpu(), O.swiglu_composed(u, g), f"torch_paras::swiglu {dt}")
    # a weight of another dtype promotes the result, as the reference's final `out * weight` does
    x, w = torch.randn(9, 64).bfloat16(), 1 + 0.02 * torch.randn(64)
    got = torch.ops.aten.rms_norm(x.to(device), [64], w.to(device), 1e-5)
    assert got.dtype == torch.float32
    want = O.binary(O.OP_MUL, O.rms_norm_composed(x, [64], None, 1e-5).float(), w.expand(9, 64).contiguous())
    assert_bit_exact(got.cpu(), want, "aten::rms_norm bf16 input, fp32 weight")


def test_composed_ops_streaming_kernels_are_exact(device):
    """The 16-bit streaming forms of aten::rms_norm and torch_paras::swiglu against the oracle's
    step-by-step narrowing: row sizes on each register tier and on the general kernel, with and
    without weight, every representable bf16 gate, tiny and huge magnitudes."""
    for dt in (torch.bfloat16, torch.float16):
        for H in (8, 264, 2048, 4096, 8192, 1000, 8200):
            x, w = (2 * torch.randn(19, H)).to(dt), (1 + 0.1 * torch.randn(H)).to(dt)
            got = torch.ops.aten.rms_norm(x.to(device), [H], w.to(device), 1e-6)
            assert_bit_exact(got.cpu(), O.rms_norm_composed(x, [H], w, 1e-6), f"aten::rms_norm {dt} H={H}")
            got = torch.ops.aten.rms_norm(x.to(device), [H], None, 1e-6)
            assert_bit_exact(got.cpu(), O.rms_norm_composed(x, [H], None, 1e-6), f"aten::rms_norm no weight {dt} H={H}")
        scale = 1e-18 if dt == torch.bfloat16 else 1e-3
        x = (scale * torch.randn(5, 512)).to(dt)
        got = torch.ops.aten.rms_norm(x.to(device), [512], None, 1e-6)
        assert_bit_exact(got.cpu(), O.rms_norm_composed(x, [512], None, 1e-6), f"aten::rms_norm tiny {dt}")
        # rows with NaN, infinities of both signs, zeros and huge values: NaNs must come out as the
        # host's types write them (the conversion instructions alone would keep their payloads)
        x = torch.randn(8, 4096)
        x[0, 5] = float("nan"); x[1, 7] = float("inf"); x[2, 9] = float("-inf"); x[2, 10] = float("inf")
        x[3] = 0.0; x[4] *= 1e4 if dt == torch.float16 else 1e30; x[5, ::2] = -0.0
        x = x.to(dt)
        x[6].view(torch.int16)[3] = 0x7FA5 if dt == torch.bfloat16 else 0x7DA5          # a NaN with a payload
        w4 = (1 + 0.1 * torch.randn(4096)).to(dt)
        for wt in (w4, None):
            got = torch.ops.aten.rms_norm(x.to(device), [4096], None if wt is None else wt.to(device), 1e-6)
            assert_bit_exact(got.cpu(), O.rms_norm_composed(x, [4096], wt, 1e-6), f"aten::rms_norm special values {dt}")
        g = (4 * torch.randn(5, 1031)).to(dt)
        u = (torch.randn(5, 1031) * torch.tensor([1e-30, 1.0, 1e3, 1e-3, 30.0]).view(5, 1)).to(dt)
        got = torch.ops.torch_paras.swiglu(u.to(device), g.to(device))
        assert_bit_exact(got.cpu(), O.swiglu_composed(u, g), f"torch_paras::swiglu {dt}")
    gate = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    for xv in (1.0, -0.3, 7.25):
        x = torch.full_like(gate, xv)
        got = torch.ops.torch_paras.swiglu(x.to(device), gate.to(device))
        want = O.swiglu_composed(x, gate)
        both_nan = got.cpu().isnan() & want.isnan()
        assert torch.equal(got.cpu().view(torch.int16)[~both_nan], want.view(torch.int16)[~both_nan]), f"all gates, x={xv}"


def test_swiglu(device):
    x, gate = torch.randn(4, 32), torch.randn(4, 32)
    assert_close(torch.ops.torch_paras.swiglu(x.to(device), gate.to(device)), torch.ops.torch_paras.swiglu(x, gate), "swiglu")
    assert_close(torch.ops.torch_paras.swiglu(x.to(device), gate.to(device)), x * F.silu(gate), "swiglu manual")
    b = torch.randn(32)
    assert_close(torch.ops.torch_paras.swiglu(b.to(device), gate.to(device)), b * F.silu(gate), "swiglu broadcast")


# ---- fused ops with autograd (reference tests/test_fused_ops.py:8-70) --------------
def test_fused_forward_and_backward(device):
    from torch_paras import nn as paras_nn
    x = torch.randn(4, 8, requires_grad=True)
    w = torch.randn(8, requires_grad=True)
    ref = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w
    ref.sum().backward()
    xd, wd = x.detach().to(device).requires_grad_(), w.detach().to(device).requires_grad_()
    out = paras_nn.rms_norm(xd, wd, 1e-6)
    out.sum().backward()
    assert_close(out.detach(), ref.detach(), "rms_norm")
    assert_close(xd.grad, x.grad, "rms_norm.grad_input")
    assert_close(wd.grad, w.grad, "rms_norm.grad_weight")

    gate, up = torch.randn(4, 8, requires_grad=True), torch.randn(4, 8, requires_grad=True)
    (F.silu(gate) * up).sum().backward()
    gd, ud = gate.detach().to(device).requires_grad_(), up.detach().to(device).requires_grad_()
    res = paras_nn.swiglu(gd, ud)
    res.sum().backward()
    assert_close(res.detach(), (F.silu(gate) * up).detach(), "swiglu")
    assert_close(gd.grad, gate.grad, "swiglu.grad_gate")
    assert_close(ud.grad, up.grad, "swiglu.grad_up")

    r = torch.randn(4, 8, requires_grad=True)
    x1, x2 = r.chunk(2, dim=-1)
    torch.cat((-x2, x1), dim=-1).sum().backward()
    rd = r.detach().to(device).requires_grad_()
    rot = paras_nn.rotate_half(rd)
    rot.sum().backward()
    assert_close(rot.detach(), torch.cat((-x2, x1), dim=-1).detach(), "rotate_half")
    assert_close(rd.grad, r.grad, "rotate_half.grad")
    with pytest.raises(RuntimeError):
        paras_nn.swiglu(torch.randn(4, 8).to(device), torch.randn(4, 9).to(device))
    with pytest.raises(RuntimeError):
        paras_nn.rms_norm(torch.randn(4, 8).to(device), torch.randn(7).to(device))


def test_fused_ops_bf16_match_host_engine(device):
    from torch_paras import nn as paras_nn
    x, w = torch.randn(300, 4096).bfloat16(), (1 + 0.02 * torch.randn(4096)).bfloat16()
    out, rstd = torch.ops.paras.rms_norm(x.to(device), w.to(device), 1e-6)
    want, wrstd = O.rms_norm(x, w, 1e-6)
    assert_bit_exact(out.cpu(), want, "paras::rms_norm")
    assert_bit_exact(rstd.cpu(), wrstd, "rstd")
    g, u = torch.randn(64, 14336).bfloat16(), torch.randn(64, 14336).bfloat16()
    assert_bit_exact(paras_nn.swiglu(g.to(device), u.to(device)).cpu(), O.swiglu(g, u), "paras::swiglu")
    xs = torch.randn(64, 256).bfloat16().to(device)[:, ::2]           # strided input is made contiguous
    assert_bit_exact(torch.ops.paras.swiglu(xs, xs).cpu(), O.swiglu(xs.cpu().contiguous(), xs.cpu().contiguous()), "strided")


# ---- MoE --------------------------------------------------------------------------
def test_moe_layer(device):
    from torch_paras import nn as paras_nn
    T, E, k, H, I = 300, 8, 2, 256, 512
    dt = torch.bfloat16
    x, logits = torch.randn(T, H).to(dt), torch.randn(T, E).to(dt)
    wg, wu, wd = (0.05 * torch.randn(E, I, H)).to(dt), (0.05 * torch.randn(E, I, H)).to(dt), (0.05 * torch.randn(E, H, I)).to(dt)
    route = paras_nn.moe_route(logits.to(device), k)
    want = O.moe_route(logits, k)
    for g, w_ in zip(route, want):
        assert_bit_exact(g.cpu(), w_, "moe_route")
    out = paras_nn.moe_layer(x.to(device), logits.to(device), wg.to(device), wu.to(device), wd.to(device), k)
    ref = O.moe_ffn(x, wg, wu, wd, want[1], want[2], want[3], want[5], k, gemm="aten")
    assert out.shape == (T, H) and (out.cpu().float() - ref.float()).abs().max().item() <= 2e-2
    # a view at an odd storage offset is moved onto a 16-byte boundary for the MFMA tiles: the same bits
    shifted = torch.empty(T * H + 1, dtype=dt).to(device)[1:].view(T, H)
    shifted.copy_(x.to(device))
    again = paras_nn.moe_layer(shifted, logits.to(device), wg.to(device), wu.to(device), wd.to(device), k)
    assert_bit_exact(again.cpu(), out.cpu(), "moe_layer from a misaligned view")


# ---- copies and plumbing (reference tests/test_attention_norm_ops.py:172-216) -----
def test_copy_same_shape_dtype_cast_and_host(device):
    a, src = torch.randn(4, 5), torch.randn(4, 5)
    assert_close(a.to(device).clone().copy_(src.to(device)), a.clone().copy_(src), "copy_same_shape")
    h = torch.randn(4, 5).half()
    assert_close(a.to(device).clone().copy_(h.to(device)), a.clone().copy_(h), "copy_dtype_cast")
    d = torch.randn(4, 5).to(device)
    s = torch.randn(4, 5)
    d.copy_(s)
    assert_close(d.cpu(), s, "copy_from_host")
    with pytest.raises(RuntimeError):                    # device-to-device broadcast copy is refused, as in the reference
        torch.randn(4, 5).to(device).clone().copy_(torch.randn(5).to(device))


def test_views_strides_fill_item_and_fallback(device):
    x = torch.randn(6, 8, 10)
    d = x.to(device)
    assert_close(d.permute(2, 0, 1).contiguous(), x.permute(2, 0, 1).contiguous(), "permute+contiguous")
    assert_close(d[:, 2:6, ::3], x[:, 2:6, ::3], "slice to host")
    assert_close(d.transpose(0, 2).reshape(10, 48), x.transpose(0, 2).reshape(10, 48), "reshape copy")
    assert_close(d.view(48, 10).t(), x.view(48, 10).t(), "view/t")
    assert_close(d.to(torch.bfloat16), x.to(torch.bfloat16), "to bf16 on device")
    assert_close(d.double().float(), x, "round trip through double")
    z = torch.empty(3, 4, device=device).fill_(2.5)
    assert_close(z, torch.full((3, 4), 2.5), "fill_")
    assert_close(torch.zeros(5, dtype=torch.int64, device=device), torch.zeros(5, dtype=torch.int64), "zeros int64")
    z[:, 1].zero_()
    assert z.cpu()[:, 1].abs().sum().item() == 0 and z.cpu()[:, 0].sum().item() == 7.5
    assert d[1, 2, 3].item() == x[1, 2, 3].item()
    assert_close(torch.relu(d) + 1, torch.relu(x) + 1, "CPU fallback ops")           # unregistered ops bounce through the host
    assert_close((d @ d.transpose(1, 2)), x @ x.transpose(1, 2), "matmul fallback")
    i = torch.arange(12, device=device).view(3, 4)
    assert_close(i.t().contiguous(), torch.arange(12).view(3, 4).t().contiguous(), "int64 strided copy")


def test_threads_dispatch_concurrently(device):
    import threading
    errs = []

    def work():
        try:
            x = torch.randn(64, 512).bfloat16()
            w = torch.ones(512).bfloat16()
            for _ in range(20):
                out, _ = torch.ops.paras.rms_norm(x.to(device), w.to(device), 1e-6)
            want, _ = O.rms_norm(x, w, 1e-6)
            assert torch.equal(out.cpu().view(torch.int16), want.view(torch.int16))
        except Exception as e:  # noqa: BLE001
            errs.append(e)
    ts = [threading.Thread(target=work) for _ in range(4)]
    [t.start() for t in ts]
    [t.join() for t in ts]
    assert not errs, errs


# ---- GEMM on the device (reference: host bounce, csrc/ops/vision_ops.cpp:248-309,388-423;
# its tests compare with torch-CPU, tests/test_matmul_sort_creation_ops.py:28-98) --------
def _one_ulp(actual, expected, dtype):
    mant = 7 if dtype == torch.bfloat16 else 10
    e = expected.double()
    tol = torch.exp2(torch.floor(torch.log2(e.abs().clamp_min(2.0 ** -14))) - mant) * 1.001 + 1e-6
    err = (actual.cpu().double() - e).abs()
    assert bool((err <= tol).all()), f"worst {err.max().item():.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_linear_mm_bmm_addmm_on_device(device, dtype):
    torch.manual_seed(0)
    x, w, b = torch.randn(6, 50, 256).to(dtype), (0.05 * torch.randn(384, 256)).to(dtype), torch.randn(384).to(dtype)
    xd, wd, bd = x.to(device), w.to(device), b.to(device)
    _one_ulp(F.linear(xd, wd, bd), F.linear(x, w, b), dtype)                  # nn.Linear: weight used in place as w.t()
    _one_ulp(F.linear(xd, wd), F.linear(x, w), dtype)
    m1, m2 = torch.randn(70, 128).to(dtype), (0.1 * torch.randn(128, 200)).to(dtype)
    _one_ulp(torch.mm(m1.to(device), m2.to(device)), torch.mm(m1, m2), dtype)  # row-major mat2: one transposing copy
    s = torch.randn(70, 200).to(dtype)
    _one_ulp(torch.addmm(s.to(device), m1.to(device), m2.to(device), beta=0.5, alpha=2.0),
             torch.addmm(s, m1, m2, beta=0.5, alpha=2.0), dtype)
    a3, b3 = torch.randn(4, 33, 64).to(dtype), (0.1 * torch.randn(4, 64, 48)).to(dtype)
    _one_ulp(torch.bmm(a3.to(device), b3.to(device)), torch.bmm(a3, b3), dtype)
    q, k = torch.randn(2, 3, 40, 64).to(dtype), torch.randn(2, 3, 24, 64).to(dtype)
    _one_ulp(torch.matmul(q.to(device), k.to(device).transpose(-1, -2)), torch.matmul(q, k.transpose(-1, -2)), dtype)


def test_gemm_other_dtypes_and_shapes_stay_on_the_device(device):
    """fp32 / fp64 products and contraction sizes the MFMA kernels do not take run on the general
    device kernel (reference tolerance against torch-CPU; fp32 accumulation and one rounding for the
    16-bit dtypes, so those agree with ATen-CPU to one unit in the last place)."""
    torch.manual_seed(1)
    a, b = torch.randn(17, 30), torch.randn(30, 9)
    assert_close(torch.mm(a.to(device), b.to(device)), torch.mm(a, b), "fp32 mm")          # reference tolerance
    ad, bd = torch.randn(70, 130, dtype=torch.float64), torch.randn(130, 65, dtype=torch.float64)
    assert torch.allclose(torch.mm(ad.to(device), bd.to(device)).cpu(), torch.mm(ad, bd), rtol=1e-12, atol=1e-12)
    x, w, bias = torch.randn(5, 33, 100), torch.randn(77, 100), torch.randn(77)
    assert_close(F.linear(x.to(device), w.to(device), bias.to(device)), F.linear(x, w, bias), "fp32 linear")
    a3, b3 = torch.randn(3, 20, 31), torch.randn(3, 31, 12)
    assert_close(torch.bmm(a3.to(device), b3.to(device)), torch.bmm(a3, b3), "fp32 bmm")
    s_ = torch.randn(17, 9)
    assert_close(torch.addmm(s_.to(device), a.to(device), b.to(device), beta=0.5, alpha=2.0), torch.addmm(s_, a, b, beta=0.5, alpha=2.0), "fp32 addmm")
    for dt in (torch.bfloat16, torch.float16):
        a16, b16 = torch.randn(8, 24).to(dt), torch.randn(24, 8).to(dt)                       # K not a multiple of 64
        _one_ulp(torch.mm(a16.to(device), b16.to(device)), torch.mm(a16, b16), dt)
    with pytest.raises(RuntimeError):
        torch.mm(a.to(device), torch.randn(31, 9).to(device))
    with pytest.raises(RuntimeError, match="float dtypes"):
        torch.mm(torch.ones(4, 4, dtype=torch.int32).to(device), torch.ones(4, 4, dtype=torch.int32).to(device))


def test_linear_backward_through_device_gemm(device):
    torch.manual_seed(2)
    x, w = torch.randn(32, 128).bfloat16(), (0.1 * torch.randn(64, 128)).bfloat16()
    xd, wd = x.to(device).requires_grad_(), w.to(device).requires_grad_()
    xc, wc = x.clone().requires_grad_(), w.clone().requires_grad_()
    F.linear(xd, wd).float().pow(2).sum().backward()
    F.linear(xc, wc).float().pow(2).sum().backward()
    for got, want in ((xd.grad, xc.grad), (wd.grad, wc.grad)):
        err = (got.cpu().float() - want.float()).abs().max().item()
        assert err <= 0.02 * want.float().abs().max().item() + 1e-3, err


def test_softmax_and_topk_ops_on_device(device):
    torch.manual_seed(3)
    x = torch.randn(4, 6, 50)
    xd = x.to(device)
    for dim in (-1, 1, 0):
        assert_close(torch.softmax(xd, dim), torch.softmax(x, dim), f"softmax dim {dim}")
    h = x.half()
    out = torch.softmax(h.to(device), -1, dtype=torch.float32)           # half_to_float
    assert out.dtype == torch.float32
    assert_close(out, torch.softmax(h, -1, dtype=torch.float32), "softmax half_to_float")
    for dim, k in ((-1, 5), (1, 3)):
        v, i = torch.topk(xd, k, dim=dim)
        tv, ti = torch.topk(x, k, dim=dim)
        assert torch.equal(i.cpu(), ti) and torch.equal(v.cpu(), tv)
    v, i = torch.topk(torch.tensor([[5, 3, 5, 5, 1, 3]]).to(device), 4)  # integer dtype: host route
    assert v.cpu().tolist() == [[5, 5, 5, 3]]


def test_covered_ops_never_take_the_host_fallback():
    """With PARAS_LOG=1 the device prints every op that goes through the dispatcher's CPU fallback:
    none of the ops this build covers may appear there, in any dtype it registers."""
    import os
    import subprocess
    import sys
    code = r"""
import sys, torch, torch.nn.functional as F
sys.path.insert(0, sys.argv[1])
import torch_paras
dev = "paras:0"
for dt in (torch.bfloat16, torch.float16, torch.float32):
    q, k, v = (torch.randn(2, 4, 64, 64).to(dt).to(dev) for _ in range(3))
    F.scaled_dot_product_attention(q, k, v, is_causal=True)
    F.scaled_dot_product_attention(q, k, v, attn_mask=(torch.rand(64, 64) > 0.3).to(dev))
    x, w = torch.randn(8, 256).to(dt).to(dev), torch.randn(256).to(dt).to(dev)
    F.rms_norm(x, (256,), w, 1e-6)
    torch.ops.paras.rms_norm(x, w, 1e-6)
    torch.ops.paras.swiglu(x, x)
    torch.ops.torch_paras.swiglu(x, x)
    W = torch.randn(128, 256).to(dt).to(dev)
    F.linear(x, W)
    torch.mm(x, W.t())
    torch.bmm(x.view(2, 4, 256), W.t().expand(2, 256, 128))
    torch.softmax(x, -1)
    torch.topk(x, 2)
torch_paras.synchronize()
print("done")
"""
    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "framework-torch-paras_amd")
    env = dict(os.environ, PARAS_LOG="1")
    r = subprocess.run([sys.executable, "-c", code, root], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0 and "done" in r.stdout, r.stderr[-2000:]
    fell = sorted({line.split("for ", 1)[1].strip() for line in r.stderr.splitlines() if "falling back to CPU for" in line})
    covered = ("scaled_dot_product", "rms_norm", "swiglu", "linear", "mm", "softmax", "topk")
    bad = [op for op in fell if any(c in op for c in covered)]
    assert not bad, f"covered ops went through the host fallback: {bad} (all fallbacks: {fell})"


def test_llama_block_forward_matches_cpu(device):
    """One decoder block assembled from the ops of this build (RMSNorm, QKV / output / MLP projections,
    RoPE through rotate_half, causal GQA attention, SwiGLU), the glue (elementwise arithmetic,
    reshapes) going wherever the dispatcher sends it: the same code on `paras:0` and on the CPU."""
    from torch_paras import nn as paras_nn
    torch.manual_seed(11)
    B, S, Hd, nh, nkv, hd, I = 2, 96, 256, 4, 2, 64, 512
    dt = torch.bfloat16
    W = {n: (torch.randn(*shp) * 0.05).to(dt) for n, shp in
         dict(q=(nh * hd, Hd), k=(nkv * hd, Hd), v=(nkv * hd, Hd), o=(Hd, nh * hd), g=(I, Hd), u=(I, Hd), d=(Hd, I)).items()}
    n1, n2 = (1 + 0.1 * torch.randn(Hd)).to(dt), (1 + 0.1 * torch.randn(Hd)).to(dt)
    x = torch.randn(B, S, Hd).to(dt)
    pos = torch.arange(S, dtype=torch.float32)
    inv = 1.0 / (10000 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd))
    ang = torch.cat([pos[:, None] * inv[None, :]] * 2, -1)
    cos, sin = ang.cos().to(dt), ang.sin().to(dt)

    def block(x, W, n1, n2, cos, sin, rot):
        h = F.rms_norm(x, (Hd,), n1, 1e-6)
        q = F.linear(h, W["q"]).view(B, S, nh, hd).transpose(1, 2)
        k = F.linear(h, W["k"]).view(B, S, nkv, hd).transpose(1, 2)
        v = F.linear(h, W["v"]).view(B, S, nkv, hd).transpose(1, 2)
        q = q * cos + rot(q) * sin
        k = k * cos + rot(k) * sin
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
        x = x + F.linear(a.transpose(1, 2).reshape(B, S, nh * hd), W["o"])
        h = F.rms_norm(x, (Hd,), n2, 1e-6)
        m = torch.ops.torch_paras.swiglu(F.linear(h, W["u"]), F.linear(h, W["g"]))
        return x + F.linear(m, W["d"])

    def rot_cpu(t):
        return torch.cat([-t[..., hd // 2:], t[..., : hd // 2]], -1)

    want = block(x, W, n1, n2, cos, sin, rot_cpu)
    to = lambda t: t.to(device)
    got = block(to(x), {n: to(w) for n, w in W.items()}, to(n1), to(n2), to(cos), to(sin), paras_nn.rotate_half)
    err = (got.cpu().float() - want.float()).abs()
    assert got.dtype == dt and got.shape == want.shape
    assert err.max().item() <= 6e-2 and err.mean().item() <= 4e-3, (err.max().item(), err.mean().item())


def test_strided_copies_and_conversions_wide_paths(device):
    """Copies whose rows are contiguous run with 16-byte elements, dense conversions eight elements
    per thread; shapes on and off those paths (odd row lengths, views that start off alignment,
    broadcast sources) must all give what the CPU gives."""
    torch.manual_seed(23)
    for dt in (torch.bfloat16, torch.float32, torch.float16):
        a = torch.randn(2, 4, 33, 64).to(dt)
        d = a.to(device)
        assert torch.equal(d.transpose(1, 2).contiguous().cpu(), a.transpose(1, 2).contiguous())      # head transpose
        assert torch.equal(d[..., 8:40].contiguous().cpu(), a[..., 8:40].contiguous())                # slice of rows
        assert torch.equal(d[..., 3:40].contiguous().cpu(), a[..., 3:40].contiguous())                # rows off alignment
        assert torch.equal(d[:, :, ::2].contiguous().cpu(), a[:, :, ::2].contiguous())                # strided rows
        assert torch.equal(d.permute(3, 0, 1, 2).contiguous().cpu(), a.permute(3, 0, 1, 2).contiguous())   # no contiguous rows
        assert torch.equal(d[:, :1].expand(2, 4, 33, 64).contiguous().cpu(), a[:, :1].expand(2, 4, 33, 64).contiguous())
        for to in (torch.float32, torch.bfloat16, torch.float16, torch.float64):
            assert torch.equal(d.to(to).cpu(), a.to(to)), f"{dt} -> {to}"
            b = torch.randn(1003).to(dt)
            assert torch.equal(b.to(device).to(to).cpu(), b.to(to))
            assert torch.equal(b.to(device)[1:].to(to).cpu(), b[1:].to(to))                            # unaligned start
    dst = torch.zeros(4, 6, 16, dtype=torch.bfloat16).to(device)
    src = torch.randn(4, 3, 16).bfloat16()
    dst[:, 1::2] = src.to(device)                                                                        # strided destination
    ref = torch.zeros(4, 6, 16, dtype=torch.bfloat16)
    ref[:, 1::2] = src
    assert torch.equal(dst.cpu(), ref)


def test_elementwise_binary_ops_on_device_match_the_host_engine(device):
    """add / sub / mul / div of float tensors run on the device and give the bits of the reference's
    binary_kernel (double evaluation, one narrowing): same shape, broadcast rows, broadcast single
    values, Python numbers, alpha, general strides, in-place forms; wide exponent gaps for the
    fp32 add that stands in for the double one."""
    torch.manual_seed(29)
    ops = ((torch.add, O.OP_ADD), (torch.sub, O.OP_SUB), (torch.mul, O.OP_MUL), (torch.div, O.OP_DIV))
    for dt in (torch.bfloat16, torch.float16, torch.float32, torch.float64):
        a = torch.randn(3, 5, 16, 64).to(dt)
        scale = torch.tensor([1e-6, 1.0, 3e4]).view(3, 1, 1, 1) if dt != torch.float16 else torch.tensor([1e-3, 1.0, 30.0]).view(3, 1, 1, 1)
        b = (torch.randn(3, 5, 16, 64) * scale).to(dt)
        row = torch.randn(16, 64).to(dt)
        col = torch.randn(5, 1, 1).to(dt)
        odd = torch.randn(3, 5, 16, 7).to(dt)
        for fn, code in ops:
            for x, y in ((a, b), (a, row), (a, col), (odd, odd.flip(-1)), (a.transpose(1, 2), b.transpose(1, 2))):
                got = fn(x.to(device), y.to(device)).cpu()
                assert_bit_exact(got, O.binary(code, x, y), f"{fn.__name__} {dt} {tuple(x.shape)} {tuple(y.shape)}")
            got = fn(a.to(device), 0.3).cpu()
            assert_bit_exact(got, O.binary_scalar(code, a, 0.3), f"{fn.__name__} {dt} with a number")
        assert_bit_exact(torch.add(a.to(device), b.to(device), alpha=0.25).cpu(), O.binary(O.OP_ADD, a, b, 0.25), f"add alpha {dt}")
        assert_bit_exact((2.0 * a.to(device)).cpu(), O.binary_scalar(O.OP_MUL, a, 2.0), f"number * tensor {dt}")
        d = a.to(device).clone()
        d += b.to(device)
        d *= row.to(device)
        assert_bit_exact(d.cpu(), O.binary(O.OP_MUL, O.binary(O.OP_ADD, a, b), row), f"in-place {dt}")
        # signed zeros, infinities and NaNs (with payloads) keep the host's bits: -0 * x = -0, and a NaN
        # comes out as the host's 16-bit types write it
        z = torch.tensor([0.0, -0.0, 1.5, -2.0, float("inf"), float("-inf"), float("nan"), 1e-30]).to(dt)
        zz, tt = z.view(8, 1).expand(8, 8).contiguous(), z.view(1, 8).expand(8, 8).contiguous()
        for fn, code in ops:
            got, want = fn(zz.to(device), tt.to(device)).cpu(), O.binary(code, zz, tt)
            assert_bit_exact(got, want, f"{fn.__name__} {dt} special values")
    # integer tensors take the host route; a promoting mix of float dtypes is computed on the device: same values as the CPU
    i = torch.arange(12).view(3, 4)
    assert torch.equal((i.to(device) + i.to(device)).cpu(), i + i)
    m = torch.randn(4, 4).bfloat16()
    f = torch.randn(4, 4)
    assert torch.equal((m.to(device) + f.to(device)).cpu(), m + f)


def test_binary_ops_of_two_float_dtypes_and_in_place_forms(device):
    """Two float dtypes: both operands are converted to the promoted dtype and the op is evaluated there
    (the reference's to_compute, csrc/ops/pointwise_ops.cpp:55-69).  The in-place forms keep self's
    dtype and storage: `other` is narrowed to it first (binary_kernel(self, other, self), :292-296),
    so the result differs from torch's CPU one, which adds in float before narrowing.  Operands that
    overlap self in memory still give the value of the out-of-place op; an integer self with a float
    other raises as torch does."""
    torch.manual_seed(41)
    codes = (("add", O.OP_ADD), ("sub", O.OP_SUB), ("mul", O.OP_MUL), ("div", O.OP_DIV))
    bf, h, f, d = torch.randn(6, 40).bfloat16(), torch.randn(6, 40).half(), torch.randn(6, 40), torch.randn(6, 40).double()
    for name, code in codes:
        for x, y in ((bf, f), (h, bf), (f, d), (h, f), (f, bf)):
            common = torch.result_type(x, y)
            got = getattr(torch, name)(x.to(device), y.to(device))
            assert got.dtype == common
            assert_bit_exact(got.cpu(), O.binary(code, x.to(common), y.to(common)), f"{name} {x.dtype} {y.dtype}")
            xd = x.to(device)
            where = xd.data_ptr()
            getattr(xd, name + "_")(y.to(device))
            assert xd.data_ptr() == where and xd.dtype == x.dtype
            assert_bit_exact(xd.cpu(), O.binary(code, x, y.to(x.dtype)), f"{name}_ {x.dtype} by {y.dtype}")
    # a zero-dim device tensor of a wider dtype does not promote
    got = h.to(device) * torch.tensor(0.3, dtype=torch.float64).to(device)
    assert got.dtype == torch.float16
    assert_bit_exact(got.cpu(), O.binary_scalar(O.OP_MUL, h, 0.3), "f16 * 0-dim f64")
    # self read and written by the same call
    x = torch.randn(6, 8).bfloat16()
    xd = x.to(device)
    xd += xd
    assert_bit_exact(xd.cpu(), O.binary(O.OP_ADD, x, x), "x += x")
    x = torch.randn(6, 8)
    xd = x.to(device)
    xd[1:] += xd[:-1]
    want = x.clone()
    want[1:] = x[1:] + x[:-1]
    assert torch.equal(xd.cpu(), want)
    xd = x.to(device)
    xd.t().mul_(xd.t())
    assert torch.equal(xd.cpu(), x * x)
    with pytest.raises(RuntimeError, match="can't be cast"):
        torch.arange(6).to(device).add_(torch.randn(6).to(device))
    with pytest.raises(RuntimeError, match="broadcast shape"):
        torch.randn(5).to(device).add_(torch.randn(4, 5).to(device))


def test_decoder_block_runs_without_any_host_fallback():
    """Between its inputs and its output a bf16 decoder block (norms, projections, RoPE, causal GQA
    attention, SwiGLU MLP, residuals) must not send a single op through the CPU fallback."""
    import os
    import subprocess
    import sys
    code = r"""
import sys, torch, torch.nn.functional as F
sys.path.insert(0, sys.argv[1])
import torch_paras
from torch_paras import nn as pn
dev = "paras:0"
torch.manual_seed(0)
B, S, Hd, nh, nkv, hd, I = 2, 96, 256, 4, 2, 64, 512
to = lambda t: t.to(torch.bfloat16).to(dev)
W = {n: to(torch.randn(*shp) * 0.05) for n, shp in dict(q=(nh*hd, Hd), k=(nkv*hd, Hd), v=(nkv*hd, Hd), o=(Hd, nh*hd), g=(I, Hd), u=(I, Hd), d=(Hd, I)).items()}
n1, n2 = to(torch.ones(Hd)), to(torch.ones(Hd))
x, cos, sin = to(torch.randn(B, S, Hd)), to(torch.randn(S, hd)), to(torch.randn(S, hd))
print("=== block starts", file=sys.stderr, flush=True)
h = F.rms_norm(x, (Hd,), n1, 1e-6)
q = F.linear(h, W["q"]).view(B, S, nh, hd).transpose(1, 2)
k = F.linear(h, W["k"]).view(B, S, nkv, hd).transpose(1, 2)
v = F.linear(h, W["v"]).view(B, S, nkv, hd).transpose(1, 2)
q = q * cos + pn.rotate_half(q) * sin
k = k * cos + pn.rotate_half(k) * sin
a = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
x = x + F.linear(a.transpose(1, 2).reshape(B, S, nh * hd), W["o"])
h = F.rms_norm(x, (Hd,), n2, 1e-6)
m = torch.ops.torch_paras.swiglu(F.linear(h, W["u"]), F.linear(h, W["g"]))
y = x * 0.5 + F.linear(m, W["d"])
torch_paras.synchronize()
print("=== block ends", file=sys.stderr, flush=True)
print("done")
"""
    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "framework-torch-paras_amd")
    r = subprocess.run([sys.executable, "-c", code, root], capture_output=True, text=True, env=dict(os.environ, PARAS_LOG="1"), timeout=300)
    assert r.returncode == 0 and "done" in r.stdout, r.stderr[-2000:]
    err = r.stderr
    inside = err[err.index("=== block starts"):err.index("=== block ends")]
    fell = sorted({line.split("for ", 1)[1].strip() for line in inside.splitlines() if "falling back to CPU for" in line})
    assert not fell, f"ops of the block went through the host: {fell}"


def test_cat_index_select_and_embedding_on_device(device):
    """KV-cache appends, row gathers and embedding lookups stay on the device and equal the CPU's."""
    torch.manual_seed(37)
    for dt in (torch.bfloat16, torch.float32, torch.int64):
        mk = (lambda *s: torch.randn(*s).to(dt)) if dt.is_floating_point else (lambda *s: torch.randint(-50, 50, s))
        a, b, c = mk(2, 4, 7, 16), mk(2, 4, 1, 16), mk(2, 4, 3, 16)
        for dim in (2, -2):
            assert torch.equal(torch.cat([a.to(device), b.to(device), c.to(device)], dim).cpu(), torch.cat([a, b, c], dim))
        assert torch.equal(torch.cat([a.to(device), a.to(device)], 0).cpu(), torch.cat([a, a], 0))
        assert torch.equal(torch.cat([a.to(device), a.to(device)], -1).cpu(), torch.cat([a, a], -1))
        assert torch.equal(torch.cat([a.to(device).transpose(1, 2), a.to(device).transpose(1, 2)], 1).cpu(),
                           torch.cat([a.transpose(1, 2), a.transpose(1, 2)], 1))
        t = mk(5, 6, 9)
        idx = torch.tensor([4, 0, 0, 3, 1])
        for dim in (0, 1, 2, -1):
            n = t.size(dim)
            ix = idx % n
            assert torch.equal(torch.index_select(t.to(device), dim, ix.to(device)).cpu(), torch.index_select(t, dim, ix)), f"{dt} dim {dim}"
        assert torch.equal(torch.index_select(t.to(device), 0, torch.tensor(2).to(device)).cpu(), torch.index_select(t, 0, torch.tensor(2)))
    w = torch.randn(1000, 64).bfloat16()
    tok = torch.randint(0, 1000, (3, 17))
    assert torch.equal(F.embedding(tok.to(device), w.to(device)).cpu(), F.embedding(tok, w))
    w33 = torch.randn(50, 33).half()                                       # rows that are not a multiple of 16 bytes
    assert torch.equal(F.embedding(tok.to(device) % 50, w33.to(device)).cpu(), F.embedding(tok % 50, w33))
    with pytest.raises(RuntimeError):
        torch.cat([torch.zeros(2, 3).to(device), torch.zeros(2, 4).to(device)], 0)


# ---- arguments on the wrong device raise on the host, before any launch ------------
def test_host_tensor_mixed_into_a_device_op_raises(device):
    """The dispatcher picks the device kernel as soon as one argument is on the device; a host
    pointer must never reach a HIP kernel."""
    import torch_paras  # noqa: F401
    bf = torch.bfloat16
    x, w = torch.randn(8, 64).to(bf), torch.randn(64).to(bf)
    dx, dw = x.to(device), w.to(device)
    cases = [
        lambda: torch.mm(dx, torch.randn(64, 16).to(bf)),
        lambda: torch.bmm(dx[None], torch.randn(1, 64, 16).to(bf)),
        lambda: torch.addmm(torch.randn(16).to(bf), dx, torch.randn(64, 16).to(bf).to(device)),
        lambda: torch.ops.paras.rms_norm(dx, w, 1e-6),
        lambda: torch.ops.paras.rms_norm_backward(dx, dx, w, torch.ones(8).to(device)),
        lambda: torch.ops.paras.rms_norm_backward(dx, dx, dw, torch.ones(8)),
        lambda: torch.ops.paras.swiglu(dx, x),
        lambda: torch.ops.paras.swiglu_backward(dx, x, dx),
        lambda: torch.ops.aten.rms_norm(dx, [64], w, 1e-6),
        lambda: torch.ops.torch_paras.swiglu(dx, x),
        lambda: torch.ops.aten._scaled_dot_product_attention_math(dx.view(1, 1, 8, 64), x.view(1, 1, 8, 64), dx.view(1, 1, 8, 64)),
        lambda: F.scaled_dot_product_attention(dx.view(1, 1, 8, 64), dx.view(1, 1, 8, 64), x.view(1, 1, 8, 64)),
    ]
    for i, fn in enumerate(cases):
        with pytest.raises(RuntimeError):
            fn()
            pytest.fail(f"case {i} did not raise")
    # MoE: weights on the host, and weights of another dtype than x
    T, E, k, H, I = 16, 2, 1, 64, 64
    xm = torch.randn(T, H).to(bf).to(device)
    route = torch.ops.paras.moe_route(torch.randn(T, E).to(bf).to(device), k)
    wg = torch.randn(E, I, H).to(bf)
    wd = torch.randn(E, H, I).to(bf)
    with pytest.raises(RuntimeError):
        torch.ops.paras.moe_ffn(xm, wg, wg.to(device), wd.to(device), route[1], route[2], route[3], route[5], k)
    with pytest.raises(RuntimeError, match="dtype"):
        torch.ops.paras.moe_ffn(xm, wg.float().to(device), wg.to(device), wd.to(device), route[1], route[2], route[3], route[5], k)


def test_sdpa_fused_path_honours_enable_gqa(device):
    """Fewer key/value heads without enable_gqa fail as in the reference (its matmul cannot
    broadcast 8 heads against 2); with the flag the fused op maps the heads."""
    q, k = torch.randn(1, 8, 16, 64).bfloat16().to(device), torch.randn(1, 2, 16, 64).bfloat16().to(device)
    with pytest.raises(RuntimeError):
        F.scaled_dot_product_attention(q, k, k, enable_gqa=False)
    out = F.scaled_dot_product_attention(q, k, k, enable_gqa=True)
    ref = F.scaled_dot_product_attention(q.cpu().float(), k.cpu().float(), k.cpu().float(), enable_gqa=True)
    assert (out.cpu().float() - ref).abs().max().item() <= 2e-2


def test_device_to_host_copy_broadcasts(device):
    src = torch.randn(5)
    dst = torch.zeros(3, 5)
    dst.copy_(src.to(device))
    assert torch.equal(dst, src.expand(3, 5))
    dst16 = torch.zeros(3, 5, dtype=torch.bfloat16)
    dst16.copy_(src.to(device))
    assert torch.equal(dst16, src.bfloat16().expand(3, 5))


def test_reference_device_numbering_on_the_gpu():
    """PARAS_DEVICE_BASE=1 with a GPU present: ops run on `paras:1`, `paras:0` raises."""
    from test_package_cpu import test_reference_device_numbering_is_an_opt_in
    test_reference_device_numbering_is_an_opt_in()


def test_empty_and_degenerate_shapes_match_the_cpu(device):
    """Zero-sized batches, rows, key lengths and contraction sizes, rank-3 and rank-5 attention
    inputs, one-element and zero-dimensional operands: same shapes, dtypes and values as torch's
    CPU ops (the reference's tests compare with torch-CPU the same way)."""
    sd = F.scaled_dot_product_attention

    def first(r):
        return r[0] if isinstance(r, (tuple, list)) else r

    def same(name, fn, *args):
        want = first(fn(*args))
        got = first(fn(*[a.to(device) if torch.is_tensor(a) else a for a in args])).cpu()
        assert got.shape == want.shape and got.dtype == want.dtype, f"{name}: {tuple(got.shape)} {got.dtype} vs {tuple(want.shape)} {want.dtype}"
        assert torch.allclose(got.float(), want.float(), rtol=2e-2, atol=2e-2, equal_nan=True), name

    for dt in (torch.bfloat16, torch.float32):
        z = lambda *s: torch.zeros(*s, dtype=dt)
        r = lambda *s: torch.randn(*s).to(dt)
        same(f"sdpa Lq=0 {dt}", sd, z(1, 2, 0, 16), r(1, 2, 5, 16), r(1, 2, 5, 16))
        same(f"sdpa Lk=0 {dt}", sd, r(1, 2, 3, 16), z(1, 2, 0, 16), z(1, 2, 0, 16))
        same(f"sdpa B=0 {dt}", sd, z(0, 2, 3, 16), z(0, 2, 3, 16), z(0, 2, 3, 16))
        same(f"sdpa D=1 {dt}", sd, r(1, 2, 3, 1), r(1, 2, 4, 1), r(1, 2, 4, 1))
        same(f"sdpa rank 3 {dt}", sd, r(2, 3, 16), r(2, 4, 16), r(2, 4, 16))
        same(f"sdpa rank 5 {dt}", sd, r(2, 2, 3, 5, 16), r(2, 2, 3, 7, 16), r(2, 2, 3, 7, 16))
        same(f"sdpa one key, causal {dt}", lambda q, k, v: sd(q, k, v, is_causal=True), r(1, 2, 5, 128), r(1, 2, 1, 128), r(1, 2, 1, 128))
        same(f"sdpa D=256 {dt}", sd, r(1, 2, 9, 256), r(1, 2, 11, 256), r(1, 2, 11, 256))
        same(f"mm K=0 {dt}", torch.mm, z(3, 0), z(0, 4))
        same(f"mm M=0 {dt}", torch.mm, z(0, 8), r(8, 4))
        same(f"mm 1x1 {dt}", torch.mm, r(1, 1), r(1, 1))
        same(f"bmm empty batch {dt}", torch.bmm, z(0, 3, 4), z(0, 4, 5))
        same(f"bmm K=0 {dt}", torch.bmm, z(2, 3, 0), z(2, 0, 5))
        same(f"linear of a vector {dt}", F.linear, r(64), r(5, 64), r(5))
        same(f"matmul of vectors {dt}", torch.matmul, r(8), r(8))
        same(f"softmax of empty rows {dt}", lambda x: torch.softmax(x, -1), z(3, 0))
        same(f"softmax 0-d {dt}", lambda x: torch.softmax(x, 0), r(()))
        same(f"topk k=0 {dt}", lambda x: torch.topk(x, 0), r(3, 5))
        same(f"add empty {dt}", torch.add, z(0, 3), z(0, 3))
        same(f"add 0-d {dt}", torch.add, r(3, 4), r(()))
        same(f"cat with an empty piece {dt}", lambda a, b, c: torch.cat([a, b, c], 0), r(2, 3), z(0, 3), r(1, 3))
        same(f"index_select with no indices {dt}", lambda x, i: torch.index_select(x, 0, i), r(4, 3), torch.zeros(0, dtype=torch.long))
        same(f"rms_norm over two dims {dt}", lambda x, w: F.rms_norm(x, [3, 16], w, 1e-5), r(2, 3, 16), r(3, 16))
    lg = torch.zeros(0, 8).to(device)
    topi, topw, order, inverse, counts, offsets = torch.ops.paras.moe_route(lg, 2)
    assert topi.shape == (0, 2) and counts.cpu().tolist() == [0] * 8 and offsets.cpu().tolist() == [0] * 9
    out, rstd = torch.ops.paras.rms_norm(torch.zeros(0, 64).to(device), torch.ones(64).to(device), 1e-6)
    assert out.shape == (0, 64) and rstd.numel() == 0
