"""GPU parity of scaled-dot-product attention through the C ABI.

Bars: fp32 within 1e-5 relative (max |a-b| / max |b|); bf16 / fp16 within 2e-2
absolute of the host-engine oracle; the generic kernel additionally reproduces
the host engine's softmax weights bit for bit (it narrows at the same points).
"""
import math

import pytest
import torch

import capi
import oracle as O
from conftest import assert_bit_exact
from golden_util import DTYPE_TAGS, case

pytestmark = pytest.mark.gpu
ABS_16BIT = 2e-2
REL_F32 = 1e-5


def run(q, k, v, **kw):
    kw = {a: (b.cuda() if torch.is_tensor(b) else b) for a, b in kw.items()}
    return capi.sdpa(q.cuda(), k.cuda(), v.cuda(), **kw)


def rel_err(a, b):
    return ((a.double().cpu() - b.double()).abs().max() / b.double().abs().max()).item()


def max_abs(a, b):
    return (a.double().cpu() - b.double()).abs().max().item()


def test_config1_fp32_causal():
    """BASELINE config 1: B=1 H=8 S=128 D=64 fp32, N(0,1), seed 0, scale 1/sqrt(D)."""
    q, k, v = torch.randn(1, 8, 128, 64), torch.randn(1, 8, 128, 64), torch.randn(1, 8, 128, 64)
    out, attn, lse, name = run(q, k, v, is_causal=True, want_attn=True, want_lse=True)
    want, wattn = O.sdpa_math(q, k, v, is_causal=True, gemm="aten")
    assert name == "generic" and out.shape == (1, 8, 128, 64)
    assert rel_err(out, want) <= REL_F32
    assert torch.allclose(out.cpu(), want, rtol=REL_F32, atol=REL_F32 * want.abs().max().item())
    assert rel_err(attn, wattn) <= REL_F32
    ref_lse = torch.logsumexp((q @ k.transpose(-1, -2) * 0.125).masked_fill(~torch.ones(128, 128).tril().bool(), -math.inf), -1)
    assert torch.allclose(lse.cpu(), ref_lse, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("tag", DTYPE_TAGS)
def test_golden_vectors_generic_kernel(tag):
    """Small heads (D=16) with every mask variant: outputs and softmax weights of
    the reference's host engine, bit for bit (fp32: 1e-5 relative, its GEMM is
    ATen's)."""
    c = case(f"sdpa_{tag}")
    q, k, v = c["q"], c["k"], c["v"]
    dtype = q.dtype
    scale32 = O.round_to_dtype(1 / math.sqrt(32), dtype)   # the op layer narrows the scale (to_compute)
    variants = {"plain": {}, "causal": dict(is_causal=True), "bool": dict(mask=c["mask"].bool()),
                "bias": dict(mask=c["bias"]), "scale": dict(scale=scale32)}
    for name, kw in variants.items():
        out, attn, _, kern = run(q, k, v, want_attn=True, **kw)
        assert kern == "generic"
        if tag == "f32":
            assert rel_err(out, c[f"out_{name}"]) <= REL_F32 and rel_err(attn, c[f"attn_{name}"]) <= REL_F32
        else:
            assert_bit_exact(attn, c[f"attn_{name}"], f"{tag} {name} weights")
            one_ulp_of_the_gemm(out, c[f"out_{name}"])
    out, _, _, kern = run(q, c["kg"], c["vg"])
    if tag == "f32":
        assert kern == "generic" and rel_err(out, c["out_gqa"]) <= REL_F32
    else:
        # no weights asked for and 16 bits: the head size is padded to 64 and the flash kernel runs
        assert kern == "padded_mfma" and max_abs(out, c["out_gqa"]) <= ABS_16BIT


@pytest.mark.parametrize("tag", ("bf16", "f16"))
def test_golden_vectors_mfma_kernels(tag):
    c = case(f"sdpa_d128_{tag}")
    out, _, _, kern = run(c["q"], c["k"], c["v"], is_causal=True)
    assert kern.startswith("flash_mfma") and max_abs(out, c["out_causal"]) <= ABS_16BIT
    out, _, _, kern = run(c["q"], c["k"], c["v"])
    assert kern.startswith("flash_mfma") and max_abs(out, c["out_plain"]) <= ABS_16BIT
    d = case(f"sdpa_decode_{tag}")
    out, _, _, kern = run(d["q"], c["k"], c["v"])
    assert kern == "decode_split" and max_abs(out, d["out"]) <= ABS_16BIT


def one_ulp_of_the_gemm(out, want):
    """The output is a GEMM of the (bit-identical) weights with V: ATen sums in
    fp32 in its own order, the kernel in fp64, so a few results land on the
    other side of a 16-bit rounding boundary.  At most one ulp, at most 1 %."""
    mant = 7 if want.dtype == torch.bfloat16 else 10
    a, b = out.double().cpu(), want.double()
    ulp = 2.0 ** (torch.floor(torch.log2(b.abs().clamp_min(1e-30))) - mant)
    assert bool(((a - b).abs() <= ulp * 1.001).all())
    assert float((a != b).double().mean()) <= 0.01


FLASH_SHAPES = [  # B, Hq, Hkv, Lq, Lk, D, causal
    (1, 2, 2, 128, 128, 128, True), (2, 4, 2, 200, 200, 128, True), (1, 2, 1, 130, 77, 64, False),
    (1, 8, 8, 256, 256, 64, True), (1, 2, 2, 64, 300, 128, True), (1, 4, 4, 300, 64, 128, True),
    (2, 2, 2, 512, 512, 128, False), (1, 1, 1, 17, 1, 128, False), (3, 5, 5, 129, 191, 64, True),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", FLASH_SHAPES)
def test_flash_matches_oracle(dtype, shape):
    B, Hq, Hkv, Lq, Lk, D, causal = shape
    q, k, v = torch.randn(B, Hq, Lq, D).to(dtype), torch.randn(B, Hkv, Lk, D).to(dtype), torch.randn(B, Hkv, Lk, D).to(dtype)
    out, _, lse, kern = run(q, k, v, is_causal=causal, want_lse=True)
    want, _ = O.sdpa_math(q, k, v, is_causal=causal, enable_gqa=True, gemm="aten")
    assert kern.startswith("flash_mfma")
    assert max_abs(out, want) <= ABS_16BIT, f"{shape} {dtype}"
    rep = Hq // Hkv
    s = (q.float() @ k.float().repeat_interleave(rep, 1).transpose(-1, -2)) / math.sqrt(D)
    if causal:
        s = s.masked_fill(~torch.ones(Lq, Lk).tril().bool(), -math.inf)
    # Scores are accumulated in fp32 from the unmodified operands and the row denominator is
    # summed from the unrounded exponentials, so the log-sum-exp is good to fp32 round-off.
    tol = 2e-4
    assert torch.allclose(lse.cpu(), torch.logsumexp(s, -1), rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_flash_accuracy_with_large_scores(dtype):
    """Inputs twice and four times the usual magnitude (score spread x4 / x16): the error against
    the exact fp64 result must stay that of rounding P and O to the operand type.  Rounding a
    pre-scaled q or k instead of scaling the fp32 scores would double it and show up in the
    log-sum-exp first."""
    torch.manual_seed(4)
    B, H, S, D = 1, 4, 1024, 128
    for mag, bar in ((2.0, 1.1e-3), (4.0, 1.3e-3)):          # mean absolute error, bf16; f16 an eighth of it
        q, k = (mag * torch.randn(B, H, S, D)).to(dtype), (mag * torch.randn(B, H, S, D)).to(dtype)
        v = torch.randn(B, H, S, D).to(dtype)
        for causal in (True, False):
            out, _, lse, kern = run(q, k, v, is_causal=causal, want_lse=True)
            assert kern.startswith("flash_mfma")
            s = (q.double() @ k.double().transpose(-1, -2)) / math.sqrt(D)
            if causal:
                s = s.masked_fill(~torch.ones(S, S).tril().bool(), -math.inf)
            want = torch.softmax(s, -1) @ v.double()
            err = (out.double().cpu() - want).abs()
            assert err.mean().item() <= (bar if dtype == torch.bfloat16 else bar / 8), f"mag {mag} causal {causal}: {err.mean().item()}"
            assert err.max().item() <= (4e-2 if dtype == torch.bfloat16 else 5e-3)   # about one unit in the last place of |out| <= 4
            assert torch.allclose(lse.double().cpu(), torch.logsumexp(s, -1), rtol=0, atol=5e-4)


def test_flash_strided_inputs_and_explicit_scale():
    """q/k/v as views of a packed [B, L, 3, H, D] projection (no copy)."""
    B, L, H, D = 2, 160, 4, 128
    qkv = torch.randn(B, L, 3, H, D).bfloat16()
    q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    dq = qkv.cuda()
    dqv, dkv, dvv = (dq[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    out, _, _, kern = capi.sdpa(dqv, dkv, dvv, is_causal=True, scale=0.05)
    want, _ = O.sdpa_math(q.contiguous(), k.contiguous(), v.contiguous(), is_causal=True, scale=0.05, gemm="aten")
    assert kern.startswith("flash_mfma") and max_abs(out, want) <= ABS_16BIT


@pytest.mark.parametrize("Lk", [77, 191, 300])
def test_flash_never_reads_past_the_last_key(Lk):
    """K / V as views of larger buffers whose rows past Lk hold NaN: the tiles that hang over the
    end of K must be completed with zeros, not with what lies behind the last key."""
    B, H, Lq, D = 2, 3, 200, 128
    q = torch.randn(B, H, Lq, D).bfloat16()
    k, v = torch.randn(B, H, Lk, D).bfloat16(), torch.randn(B, H, Lk, D).bfloat16()
    kbuf = torch.full((B, H, Lk + 130, D), float("nan"), dtype=torch.bfloat16, device="cuda")
    vbuf = torch.full((B, H, Lk + 130, D), float("nan"), dtype=torch.bfloat16, device="cuda")
    kbuf[:, :, :Lk], vbuf[:, :, :Lk] = k.cuda(), v.cuda()
    for causal in (False, True):
        out, _, _, kern = capi.sdpa(q.cuda(), kbuf[:, :, :Lk], vbuf[:, :, :Lk], is_causal=causal)
        want, _ = O.sdpa_math(q, k, v, is_causal=causal, gemm="aten")
        assert kern.startswith("flash_mfma")
        assert bool(torch.isfinite(out).all()) and max_abs(out, want) <= ABS_16BIT


def test_flash_broadcast_key_rows():
    """Row stride 0 (one key / value row expanded over Lk): every key is the same row."""
    B, H, Lq, Lk, D = 1, 2, 96, 150, 64
    q = torch.randn(B, H, Lq, D).half()
    k1, v1 = torch.randn(B, H, 1, D).half(), torch.randn(B, H, 1, D).half()
    out, _, _, kern = capi.sdpa(q.cuda(), k1.cuda().expand(B, H, Lk, D), v1.cuda().expand(B, H, Lk, D), is_causal=False)
    want, _ = O.sdpa_math(q, k1.expand(B, H, Lk, D).contiguous(), v1.expand(B, H, Lk, D).contiguous(), gemm="aten")
    assert kern.startswith("flash_mfma") and max_abs(out, want) <= ABS_16BIT


def test_flash_random_shapes_layouts_and_padding():
    """Forty seeded random cases (ragged lengths around the 32 / 64 / 128 tile edges, GQA ratios,
    [B,L,H,D] views, rows embedded in NaN-filled buffers, explicit scales) against an fp32 torch
    evaluation of softmax(q k^T s + causal) v on the same device: the tolerance is the 16-bit bar."""
    import random
    rng = random.Random(1)
    g = torch.Generator(device="cuda").manual_seed(1)

    def rnd(*shape, dt):
        return torch.randn(*shape, device="cuda", generator=g).to(dt)

    for _ in range(40):
        D, dt = rng.choice([64, 128, 256]), rng.choice([torch.bfloat16, torch.float16])
        Hkv, rep, B = rng.choice([1, 2, 3, 4]), rng.choice([1, 2, 4]), rng.choice([1, 2, 3])
        Hq = Hkv * rep
        Lq = rng.choice([2, 5, 31, 32, 33, 64, 100, 127, 128, 129, 200, 255, 256, 257, 384, 500, 513])
        Lk = rng.choice([2, 31, 32, 33, 63, 64, 65, 96, 100, 127, 128, 129, 160, 191, 192, 193, 255, 256, 300, 511, 512, 640])
        causal, layout, scale = rng.random() < 0.6, rng.choice(["bhld", "blhd", "padded"]), rng.choice([None, 0.05, 0.2])
        if layout == "bhld":
            q, k, v = rnd(B, Hq, Lq, D, dt=dt), rnd(B, Hkv, Lk, D, dt=dt), rnd(B, Hkv, Lk, D, dt=dt)
        elif layout == "blhd":
            q, k, v = (rnd(B, L, H, D, dt=dt).permute(0, 2, 1, 3) for L, H in ((Lq, Hq), (Lk, Hkv), (Lk, Hkv)))
        else:
            q = rnd(B, Hq, Lq, D + 8, dt=dt)[..., :D]
            kb = torch.full((B, Hkv, Lk + 70, D + 16), float("nan"), device="cuda", dtype=dt)
            vb = torch.full((B, Hkv, Lk + 70, D + 16), float("nan"), device="cuda", dtype=dt)
            kb[:, :, :Lk, :D], vb[:, :, :Lk, :D] = rnd(B, Hkv, Lk, D, dt=dt), rnd(B, Hkv, Lk, D, dt=dt)
            k, v = kb[:, :, :Lk, :D], vb[:, :, :Lk, :D]
        out, _, _, kern = capi.sdpa(q, k, v, is_causal=causal, scale=scale)
        s = (q.float() @ k.float().repeat_interleave(rep, 1).transpose(-1, -2)) * (scale if scale is not None else 1 / math.sqrt(D))
        if causal:
            s = s.masked_fill(~torch.ones(Lq, Lk, device="cuda").tril().bool(), -math.inf)
        want = torch.softmax(s, -1) @ v.float().repeat_interleave(rep, 1)
        case_id = f"B={B} Hq={Hq} Hkv={Hkv} Lq={Lq} Lk={Lk} D={D} {dt} causal={causal} {layout} scale={scale}"
        assert kern in ("flash_mfma", "flash_mfma_wide", "decode_split"), case_id     # a handful of queries goes to the decode kernel
        assert bool(torch.isfinite(out).all()) and float((out.float() - want).abs().max()) <= ABS_16BIT, case_id


MASK_SHAPES = [  # B, Hq, Hkv, Lq, Lk, D, mask shape
    (2, 4, 4, 200, 200, 128, (2, 1, 1, 200)),      # key-padding mask, broadcast over heads and queries
    (1, 4, 2, 130, 191, 64, (1, 1, 130, 191)),     # one [Lq, Lk] pattern for every head, ragged lengths
    (2, 2, 2, 96, 333, 128, (2, 2, 96, 333)),      # a full mask
    (1, 2, 1, 257, 70, 64, (257, 70)),             # 2-D mask, GQA
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind", ["bool", "additive"])
@pytest.mark.parametrize("shape", MASK_SHAPES)
def test_flash_with_masks_matches_oracle(dtype, kind, shape):
    """Boolean and additive masks on the flash kernel, including queries whose first 64+ keys are all
    masked (the running maximum starts at -inf) and a query with no visible key at all (NaN, as the
    host softmax gives)."""
    B, Hq, Hkv, Lq, Lk, D, mshape = shape
    q, k, v = torch.randn(B, Hq, Lq, D).to(dtype), torch.randn(B, Hkv, Lk, D).to(dtype), torch.randn(B, Hkv, Lk, D).to(dtype)
    keep = torch.rand(mshape) > 0.3
    keep[..., : min(Lk - 1, 70)] &= torch.rand(mshape[:-1] + (1,)) > 0.5     # whole leading stretches masked for half the rows
    keep[..., -1] = True                                                     # ... but every query sees something
    dead_row = None
    if len(mshape) >= 2 and mshape[-2] > 1:
        dead_row = mshape[-2] // 2
        keep[..., dead_row, :] = False                                       # a query that sees nothing
    if kind == "bool":
        mask = keep
    else:
        mask = (torch.randn(mshape) * 0.5).masked_fill(~keep, -math.inf).to(dtype)
    scale = O.round_to_dtype(1 / math.sqrt(D), dtype)      # the op layer narrows the scale to the tensor type
    out, _, _, kern = run(q, k, v, mask=mask, scale=scale)
    want, _ = O.sdpa_math(q, k, v, attn_mask=mask, enable_gqa=True, gemm="aten", scale=scale)
    assert kern.startswith("flash_mfma")
    if dead_row is not None:
        assert bool(out[:, :, dead_row].isnan().all()) and bool(want[:, :, dead_row].isnan().all())
        rows = [i for i in range(Lq) if i != dead_row]
        out, want = out[:, :, rows], want[:, :, rows]
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(want).all())
    # The host engine narrows the scores to 16 bits three times before the softmax (product, scaled
    # product, sum with the mask); with part of the keys masked out a row is often decided by one or two
    # keys, and those roundings move the result by up to 2.4e-2 from softmax(q k^T s + mask) v in fp64
    # (tests/test_parity_bars_cpu.py).  The masked kernels narrow at the same three places, so they are
    # held to the host engine, not to the exact value: 1e-2 for bf16 (measured worst 0.0078 = one step
    # of a result in [1, 2)), 2.5e-3 for fp16 (measured 0.00098).
    err_oracle = (out.double().cpu() - want.double()).abs()
    bar = 1e-2 if dtype == torch.bfloat16 else 2.5e-3
    assert float(err_oracle.max()) <= bar, f"{shape} {dtype} {kind}: worst {float(err_oracle.max()):.4f}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case_", [
    # B, Hq, Hkv, Lq, Lk, causal, mask, layout
    (1, 2, 2, 128, 128, True, None, "bhld"), (2, 4, 2, 1024, 1024, True, None, "blhd"), (1, 2, 1, 1000, 1000, True, None, "bhld"),
    (1, 2, 2, 333, 777, False, None, "padded"), (1, 2, 2, 777, 333, True, None, "bhld"), (1, 3, 3, 200, 1500, False, "bool", "bhld"),
    (1, 2, 2, 130, 191, False, "add", "blhd"), (1, 1, 1, 300, 33, True, None, "bhld"), (1, 1, 1, 17, 31, False, None, "bhld"),
    (1, 8, 2, 257, 640, False, None, "bhld")])
def test_flash_head_size_256_matches_oracle(case_, dtype):
    """Heads of 256 elements on the flash kernel (one workgroup per CU: its four tiles of K and V
    fill 128 KB of LDS, a wavefront's outputs and queries its registers): causal, masks, GQA,
    ragged lengths, strided layouts; log-sum-exp against fp64."""
    B, Hq, Hkv, Lq, Lk, causal, mk, layout = case_
    D = 256
    torch.manual_seed(Lq * 7 + Lk)
    def make(H, L):          # (host tensor, the same values on the device in the layout under test)
        if layout == "blhd":
            base = torch.randn(B, L, H, D).to(dtype)
            return base.transpose(1, 2), base.cuda().transpose(1, 2)
        if layout == "padded":
            base = torch.full((B, H, L + 3, D + 16), float("nan")).to(dtype)
            base[:, :, :L, 8:8 + D] = torch.randn(B, H, L, D).to(dtype)
            return base[:, :, :L, 8:8 + D], base.cuda()[:, :, :L, 8:8 + D]
        base = torch.randn(B, H, L, D).to(dtype)
        return base, base.cuda()
    (q, dq), (k, dk), (v, dv) = make(Hq, Lq), make(Hkv, Lk), make(Hkv, Lk)
    mask = None
    if mk == "bool":
        mask = torch.rand(B, 1, Lq, Lk) > 0.3
        mask[..., 0] = True
    elif mk == "add":
        mask = (torch.randn(1, Hq, Lq, Lk) * 0.5).to(dtype)
    scale = O.round_to_dtype(1.0 / math.sqrt(D), dtype)
    out, _, lse, name = capi.sdpa(dq, dk, dv, is_causal=causal, mask=None if mask is None else mask.cuda(), scale=scale, want_lse=True)
    want, _ = O.sdpa_math(q.contiguous(), k.contiguous(), v.contiguous(), is_causal=causal, attn_mask=mask, scale=scale, enable_gqa=True, gemm="aten")
    assert name == "flash_mfma" and out.shape == (B, Hq, Lq, D)
    assert max_abs(out, want) <= (1e-2 if mk else ABS_16BIT)
    rep = Hq // Hkv
    sc = (q.double() @ k.double().repeat_interleave(rep, 1).transpose(-1, -2)) * scale
    if causal:
        sc = sc.masked_fill(~torch.ones(Lq, Lk, dtype=torch.bool).tril(), -math.inf)
    if mk == "bool":
        sc = sc.masked_fill(~mask, -math.inf)
    elif mk == "add":
        sc = sc + mask.double()
    ref_lse = torch.logsumexp(sc, -1)
    tol = 5e-4 if mk is None else 2e-2     # (the masked kernels narrow their scores as the host engine does)
    assert float((lse.double().cpu() - ref_lse).abs().max()) <= tol


def ulps_apart(a, b):
    """Distance in units of the last place between two 16-bit float tensors of one sign pattern."""
    ia, ib = a.cpu().contiguous().view(torch.int16).int(), b.cpu().contiguous().view(torch.int16).int()
    return (ia - ib).abs()


WEIGHT_SHAPES = [  # B, Hq, Hkv, Lq, Lk, D
    (1, 2, 2, 128, 128, 128), (2, 4, 2, 200, 333, 64), (1, 8, 2, 70, 1, 128), (1, 2, 1, 257, 129, 64), (1, 3, 3, 33, 700, 128),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("variant", ["plain", "causal", "bool", "additive"])
@pytest.mark.parametrize("shape", WEIGHT_SHAPES)
def test_math_op_weights_on_the_mfma_kernel(dtype, variant, shape):
    """The math op's 16-bit callers (weights returned) run on the MFMA kernel that narrows where the
    reference's composition narrows: the weights are the host engine's up to one unit in the last
    place for a small fraction of them (fp32 instead of fp64 softmax arithmetic next to a rounding
    boundary), NaN rows included, and the output is within the 2e-2 bar."""
    B, Hq, Hkv, Lq, Lk, D = shape
    q, k, v = torch.randn(B, Hq, Lq, D).to(dtype), torch.randn(B, Hkv, Lk, D).to(dtype), torch.randn(B, Hkv, Lk, D).to(dtype)
    kw = {}
    dead_row = None
    if variant == "causal":
        kw = dict(is_causal=True)
    elif variant in ("bool", "additive"):
        keep = torch.rand(B, 1, Lq, Lk) > 0.3
        keep[..., 0] = True
        if Lq > 4:
            dead_row = Lq // 2
            keep[:, :, dead_row, :] = False                       # a query that sees nothing: NaN weights and output
        kw = dict(mask=keep if variant == "bool" else (torch.randn(B, 1, Lq, Lk) * 0.5).masked_fill(~keep, -math.inf).to(dtype))
    scale = O.round_to_dtype(1 / math.sqrt(D), dtype)      # the op layer narrows the scale to the tensor type (to_compute)
    out, attn, lse, kern = run(q, k, v, want_attn=True, want_lse=True, scale=scale, **kw)
    okw = {("attn_mask" if a == "mask" else a): b for a, b in kw.items()}
    want, wattn = O.sdpa_math(q, k, v, enable_gqa=True, gemm="aten", scale=scale, **okw)
    assert kern == "math_mfma"
    assert torch.equal(attn.cpu().isnan(), wattn.isnan()) and torch.equal(out.cpu().isnan(), want.isnan())
    if dead_row is not None:
        assert bool(attn[:, :, dead_row].isnan().all())
    ok = ~wattn.isnan()
    # One unit in the last place, except where the fp32 sum of q k^T itself (accumulated in another
    # order than ATen's) rounds to the neighbouring 16-bit score: that moves a weight by a few units
    # (the last bit of a 16-bit GEMM result is not pinned by the reference).  Absolute bar 2e-2.
    d = ulps_apart(attn, wattn)[ok]
    # Measured at [1,4,4,512,512,128] causal and [1,2,2,1024,1024,128]: 3e-5 .. 3e-4 of the weights differ,
    # 5e-7 .. 1.4e-5 by more than one unit (at most 4), the output by at most 2e-3.
    assert float((d > 1).float().mean()) <= 5e-4, f"{float((d > 1).float().mean()):.2e} of the weights more than one unit apart"
    assert float((d > 0).float().mean()) <= 5e-3, f"{float((d > 0).float().mean()):.2e} of the weights differ"
    assert float((attn.cpu().double() - wattn.double()).abs()[ok].max()) <= ABS_16BIT
    oko = ~want.isnan()
    assert float((out.cpu().double() - want.double()).abs()[oko].max()) <= ABS_16BIT
    # rows of weights sum to one; log-sum-exp of the narrowed scores
    live = ~wattn.isnan().any(-1)
    assert torch.allclose(attn.cpu().float().sum(-1)[live], torch.ones_like(attn.cpu().float().sum(-1)[live]), atol=2e-2)
    assert bool(torch.isfinite(lse.cpu()[live]).all())


@pytest.mark.parametrize("kind", ["bool", "additive"])
@pytest.mark.parametrize("view", ["transposed", "every_other", "per_query"])
def test_math_op_weights_kernel_with_masks_strided_along_the_keys(kind, view):
    """The kernel that returns the weights reads its mask element by element, so any stride along
    the keys stays on it: a transposed view, every other element of a wider tensor, one value per
    query broadcast over the keys (whole rows of NaN where that value masks)."""
    B, Hq, Hkv, Lq, Lk, D = 2, 4, 2, 140, 210, 128
    dtype = torch.bfloat16
    torch.manual_seed(sum(map(ord, view + kind)))
    q, k, v = torch.randn(B, Hq, Lq, D).to(dtype), torch.randn(B, Hkv, Lk, D).to(dtype), torch.randn(B, Hkv, Lk, D).to(dtype)

    def values(*shape):
        keep = torch.rand(*shape) > 0.3
        return keep if kind == "bool" else (torch.randn(*shape) * 0.5).masked_fill(~keep, -math.inf).to(dtype)

    if view == "transposed":
        base = values(B, 1, Lk, Lq)
        host, dev = base.transpose(-1, -2), base.cuda().transpose(-1, -2)
    elif view == "every_other":
        base = values(B, Hq, Lq, 2 * Lk)
        host, dev = base[..., ::2], base.cuda()[..., ::2]
    else:
        base = values(B, 1, Lq, 1)
        host, dev = base.expand(B, 1, Lq, Lk), base.cuda().expand(B, 1, Lq, Lk)
    assert dev.stride(-1) == {"transposed": Lq, "every_other": 2, "per_query": 0}[view]
    scale = O.round_to_dtype(1 / math.sqrt(D), dtype)
    out, attn, _, kern = capi.sdpa(q.cuda(), k.cuda(), v.cuda(), mask=dev, scale=scale, want_attn=True)
    want, wattn = O.sdpa_math(q, k, v, attn_mask=host.contiguous(), enable_gqa=True, gemm="aten", scale=scale)
    assert kern == "math_mfma"
    assert torch.equal(attn.cpu().isnan(), wattn.isnan()) and torch.equal(out.cpu().isnan(), want.isnan())
    ok = ~wattn.isnan()
    d = ulps_apart(attn, wattn)[ok]
    assert float((d > 1).float().mean()) <= 5e-4 and float((d > 0).float().mean()) <= 5e-3
    assert float((attn.cpu().double() - wattn.double()).abs()[ok].max()) <= ABS_16BIT
    assert float((out.cpu().double() - want.double()).abs()[~want.isnan()].max()) <= ABS_16BIT


def test_math_op_weights_kernel_strided_inputs_and_explicit_scale():
    """Heads sliced out of a fused [B, L, 3, H, D] projection (strided q / k / v) and an explicit
    scale (narrowed to the tensor type, as the op layer hands it over)."""
    qkv = torch.randn(2, 150, 3, 4, 128).bfloat16()
    q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    dq = qkv.cuda()
    scale = O.round_to_dtype(0.0737, torch.bfloat16)
    out, attn, _, kern = capi.sdpa(*(dq[:, :, i].permute(0, 2, 1, 3) for i in range(3)), is_causal=True, scale=scale, want_attn=True)
    want, wattn = O.sdpa_math(q, k, v, is_causal=True, scale=scale, gemm="aten")
    assert kern == "math_mfma"
    d = ulps_apart(attn, wattn)
    assert float((d > 1).float().mean()) <= 5e-4 and max_abs(attn, wattn) <= ABS_16BIT and max_abs(out, want) <= ABS_16BIT


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind", ["bool", "additive"])
@pytest.mark.parametrize("view", ["transposed", "every_other", "per_query", "three_keys", "transposed_64", "every_other_256"])
def test_flash_with_masks_strided_along_the_keys(dtype, kind, view):
    """Masks that are not contiguous along the keys stay on the flash kernel (read element by
    element): a transposed view (key stride Lq), every other element of a wider tensor (stride 2),
    one value per query broadcast over the keys (stride 0), and a contiguous mask over fewer keys
    than a run of four."""
    B, Hq, Hkv, Lq, Lk, D = (2, 4, 2, 150, 3, 128) if view == "three_keys" else (2, 4, 2, 150, 230, 128)
    if "_" in view and view.rsplit("_", 1)[1].isdigit():          # the same views at the other head sizes
        view, D = view.rsplit("_", 1)[0], int(view.rsplit("_", 1)[1])
    torch.manual_seed(sum(map(ord, view + kind)) + D)
    q, k, v = torch.randn(B, Hq, Lq, D).to(dtype), torch.randn(B, Hkv, Lk, D).to(dtype), torch.randn(B, Hkv, Lk, D).to(dtype)

    def values(*shape):      # what the mask holds, on the host, laid out however the view under test wants it
        keep = torch.rand(*shape) > 0.3
        return keep if kind == "bool" else (torch.randn(*shape) * 0.5).masked_fill(~keep, -math.inf).to(dtype)

    if view == "transposed":
        base = values(B, 1, Lk, Lq)
        host, dev = base.transpose(-1, -2), base.cuda().transpose(-1, -2)
    elif view == "every_other":
        base = values(B, Hq, Lq, 2 * Lk)
        host, dev = base[..., ::2], base.cuda()[..., ::2]
    elif view == "per_query":
        base = values(B, 1, Lq, 1)
        host, dev = base.expand(B, 1, Lq, Lk), base.cuda().expand(B, 1, Lq, Lk)
    else:
        base = values(B, 1, Lq, Lk)
        host, dev = base, base.cuda()
    assert dev.stride(-1) == {"transposed": Lq, "every_other": 2, "per_query": 0, "three_keys": 1}[view]
    scale = O.round_to_dtype(1 / math.sqrt(D), dtype)
    out, _, _, kern = capi.sdpa(q.cuda(), k.cuda(), v.cuda(), mask=dev, scale=scale)
    want, _ = O.sdpa_math(q, k, v, attn_mask=host.contiguous(), enable_gqa=True, gemm="aten", scale=scale)
    assert kern.startswith("flash_mfma"), kern
    # queries with no visible key: NaN on both sides; the others to the masked kernels' bar
    dead = want.isnan().any(-1)
    assert torch.equal(out.isnan().any(-1).cpu(), dead)
    err = (out.double().cpu() - want.double()).abs()[~dead]
    bar = 1e-2 if dtype == torch.bfloat16 else 2.5e-3
    if view == "three_keys":
        # with three keys a result is close to a single row of V, whose elements reach 2 to 4, where one
        # bf16 step is 0.0156: the result is one step off where the host engine's narrowed weights round
        # the other way (measured worst 0.0156); the absolute bar for 16-bit results applies
        bar = max(bar, ABS_16BIT)
    assert float(err.max()) <= bar, f"{view} {kind} {dtype}: worst {float(err.max()):.4f}"


DECODE_SHAPES = [(2, 8, 2, 1, 1000), (1, 4, 4, 1, 77), (3, 32, 8, 1, 2048), (1, 8, 2, 2, 300), (2, 16, 1, 1, 129), (1, 2, 2, 8, 5000)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", DECODE_SHAPES)
def test_decode_matches_oracle(dtype, shape):
    B, Hq, Hkv, Lq, Lk = shape
    q, k, v = torch.randn(B, Hq, Lq, 128).to(dtype), torch.randn(B, Hkv, Lk, 128).to(dtype), torch.randn(B, Hkv, Lk, 128).to(dtype)
    out, _, lse, kern = run(q, k, v, want_lse=True)
    want, _ = O.sdpa_math(q, k, v, enable_gqa=True, gemm="aten")
    assert kern == "decode_split"
    assert max_abs(out, want) <= ABS_16BIT
    s = (q.float() @ k.float().repeat_interleave(Hq // Hkv, 1).transpose(-1, -2)) / math.sqrt(128)
    assert torch.allclose(lse.cpu(), torch.logsumexp(s, -1), rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("D", [64, 256])
@pytest.mark.parametrize("shape", [(2, 8, 2, 1, 1000), (1, 16, 1, 1, 4099), (3, 4, 4, 3, 300), (1, 2, 2, 1, 31)])
def test_decode_head_sizes_64_and_256(dtype, shape, D):
    """The split-KV decode kernel at head size 64 (half as many contraction steps and output blocks
    per tile) and 256 (twice as many; one workgroup per CU, its V tiles fill 137 KB of LDS), with
    and without a key-padding mask."""
    B, Hq, Hkv, Lq, Lk = shape
    q, k, v = torch.randn(B, Hq, Lq, D).to(dtype), torch.randn(B, Hkv, Lk, D).to(dtype), torch.randn(B, Hkv, Lk, D).to(dtype)
    out, _, lse, kern = run(q, k, v, want_lse=True)
    want, _ = O.sdpa_math(q, k, v, enable_gqa=True, gemm="aten")
    assert kern == "decode_split" and max_abs(out, want) <= ABS_16BIT
    s = (q.float() @ k.float().repeat_interleave(Hq // Hkv, 1).transpose(-1, -2)) / math.sqrt(D)
    assert torch.allclose(lse.cpu(), torch.logsumexp(s, -1), rtol=1e-3, atol=1e-3)
    keep = torch.ones(B, 1, 1, Lk, dtype=torch.bool)
    keep[0, ..., Lk // 2:] = False
    out, _, _, kern = run(q, k, v, mask=keep)
    want, _ = O.sdpa_math(q, k, v, attn_mask=keep, enable_gqa=True, gemm="aten")
    assert kern == "decode_split" and max_abs(out, want) <= ABS_16BIT


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_decode_with_masks_matches_oracle(dtype):
    """Ragged batches: decode with a key-padding mask [B,1,1,Lk], a per-head additive bias
    [B,Hq,1,Lk], a [Lq,Lk] mask for two query positions, a sequence whose first 3000 keys are all
    masked (whole tiles, whole waves and whole splits without a visible key) and one with no visible
    key at all (NaN, as the reference's softmax gives)."""
    torch.manual_seed(31)
    B, Hq, Hkv, Lk = 3, 8, 2, 4000
    q, k, v = torch.randn(B, Hq, 1, 128).to(dtype), torch.randn(B, Hkv, Lk, 128).to(dtype), torch.randn(B, Hkv, Lk, 128).to(dtype)
    lengths = [4000, 1234, 77]
    keep = torch.zeros(B, 1, 1, Lk, dtype=torch.bool)
    for i, n in enumerate(lengths):
        keep[i, ..., :n] = True
    out, _, _, kern = run(q, k, v, mask=keep)
    want, _ = O.sdpa_math(q, k, v, attn_mask=keep, enable_gqa=True, gemm="aten")
    assert kern == "decode_split" and max_abs(out, want) <= ABS_16BIT
    bias = (2 * torch.randn(B, Hq, 1, Lk)).masked_fill(~keep, -math.inf).to(dtype)
    out, _, _, kern = run(q, k, v, mask=bias)
    want, _ = O.sdpa_math(q, k, v, attn_mask=bias, enable_gqa=True, gemm="aten")
    assert kern == "decode_split" and max_abs(out, want) <= ABS_16BIT       # measured: 0.0156 (bf16), 0.002 (fp16)
    q2 = torch.randn(B, Hq, 2, 128).to(dtype)
    m2 = torch.rand(2, Lk) > 0.5
    m2[:, 0] = True
    out, _, _, kern = run(q2, k, v, mask=m2)
    want, _ = O.sdpa_math(q2, k, v, attn_mask=m2, enable_gqa=True, gemm="aten")
    assert kern == "decode_split" and max_abs(out, want) <= ABS_16BIT
    late = torch.ones(B, 1, 1, Lk, dtype=torch.bool)
    late[0, ..., :3000] = False
    late[1] = False
    out, _, _, kern = run(q, k, v, mask=late)
    want, _ = O.sdpa_math(q, k, v, attn_mask=late, enable_gqa=True, gemm="aten")
    assert kern == "decode_split"
    assert bool(out[1].isnan().all()) and bool(want[1].isnan().all())
    assert max_abs(out[[0, 2]], want[[0, 2]]) <= ABS_16BIT


def test_generic_handles_odd_heads_masks_and_all_masked_rows():
    q, k, v = torch.randn(1, 3, 5, 24), torch.randn(1, 3, 9, 24), torch.randn(1, 3, 9, 40)
    out, attn, _, kern = run(q, k, v, want_attn=True)                # Dv != D
    want, wattn = O.sdpa_math(q, k, v, gemm="aten")
    assert kern == "generic" and out.shape == (1, 3, 5, 40) and rel_err(out, want) <= REL_F32
    mask = torch.ones(5, 9, dtype=torch.bool)
    mask[2] = False                                                    # a row with no visible key
    out, attn, _, _ = run(q, k, v, mask=mask, want_attn=True)
    want, wattn = O.sdpa_math(q, k, v, attn_mask=mask, gemm="aten")
    assert bool(out[:, :, 2].isnan().all()) and bool(want[:, :, 2].isnan().all())   # NaN, as the host softmax gives
    keep = [0, 1, 3, 4]
    assert rel_err(out[:, :, keep], want[:, :, keep]) <= REL_F32
    out, _, _, _ = run(q.double(), k.double(), v.double(), is_causal=True)
    want, _ = O.sdpa_math(q.double(), k.double(), v.double(), is_causal=True)
    assert rel_err(out, want) <= 1e-13


def test_error_conventions():
    q = torch.randn(1, 5, 4, 8, device="cuda")
    k = torch.randn(1, 2, 4, 8, device="cuda")
    with pytest.raises(capi.ParasError, match="multiple of key/value heads"):   # tests/test_attention_norm_ops.py:103-108
        capi.sdpa(q, k, k)
    q = torch.randn(1, 2, 4, 8, device="cuda")
    with pytest.raises(capi.ParasError, match="mutually exclusive"):
        capi.sdpa(q, k, k, mask=torch.ones(4, 4, dtype=torch.bool, device="cuda"), is_causal=True)
    out, _, _, _ = capi.sdpa(q[:, :, :0], k, k)                                   # empty query
    assert out.shape == (1, 2, 0, 8)


def test_config3_shape_properties_and_slice():
    """BASELINE config 3 (bf16 causal B=4 H=32 S=4096 D=128) at full size: a
    slice against the oracle, the whole output through properties."""
    B, H, S, D = 4, 32, 4096, 128
    q, k, v = torch.randn(B, H, S, D).bfloat16(), torch.randn(B, H, S, D).bfloat16(), torch.randn(B, H, S, D).bfloat16()
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    out, _, lse, kern = capi.sdpa(qd, kd, vd, is_causal=True, want_lse=True)
    assert kern == "flash_mfma_wide"        # 2048 tiles of 256 queries for 256 CUs
    want, _ = O.sdpa_math(q[:1, :2], k[:1, :2], v[:1, :2], is_causal=True, gemm="aten")
    assert max_abs(out[:1, :2], want) <= ABS_16BIT
    # rows 3000..3063 of the last head: causal == an explicit lower-triangular mask on those rows
    full_rows = O.sdpa_math(q[3:, 31:, 3000:3064], k[3:, 31:], v[3:, 31:],
                            attn_mask=torch.ones(S, S).tril().bool()[3000:3064], gemm="aten")[0]
    assert max_abs(out[3:, 31:, 3000:3064], full_rows) <= ABS_16BIT
    assert not bool(out.isnan().any())
    assert torch.equal(out[:, :, 0].cpu(), v[:, :, 0])                       # causal row 0 sees key 0 only
    ones, _, _, _ = capi.sdpa(qd, kd, torch.ones_like(vd), is_causal=True)   # weights sum to one
    assert (ones.float() - 1).abs().max().item() <= 2 ** -7
    # linearity in V: f(V1 + V2) == f(V1) + f(V2) up to 16-bit rounding of each term
    v2 = torch.randn(B, H, S, D).bfloat16().cuda()
    o2, _, _, _ = capi.sdpa(qd, kd, v2, is_causal=True)
    o12, _, _, _ = capi.sdpa(qd, kd, (vd.float() + v2.float()).bfloat16(), is_causal=True)
    assert (o12.float() - (out.float() + o2.float())).abs().max().item() <= 6e-2


@pytest.mark.parametrize("B,Hq,Hkv,Lq,Lk,causal,dtype", [
    (4, 32, 8, 1024, 1024, False, torch.bfloat16),      # grouped heads, two tiles per CU
    (4, 32, 32, 1100, 1300, False, torch.bfloat16),     # neither length a multiple of the tile sizes
    (5, 27, 27, 1024, 2000, False, torch.float16),      # a head count that does not divide by 8
    (1, 32, 8, 4096, 4096, True, torch.bfloat16),       # causal, two items per workgroup
    (2, 16, 4, 4100, 4200, True, torch.float16),        # causal, ragged last tile, Lq != Lk
])
def test_flash_wide_kernel_matches_oracle(B, Hq, Hkv, Lq, Lk, causal, dtype):
    """The 64-queries-per-wavefront form of the flash kernel (one workgroup per CU walking a
    list of 256-query items) at shapes where paras_sdpa_fwd picks it: sampled heads against the
    oracle, the log-sum-exp against fp64, strided inputs against contiguous ones."""
    torch.manual_seed(Lq + Lk)
    q, k, v = torch.randn(B, Hq, Lq, 128).to(dtype), torch.randn(B, Hkv, Lk, 128).to(dtype), torch.randn(B, Hkv, Lk, 128).to(dtype)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    out, _, lse, kern = capi.sdpa(qd, kd, vd, is_causal=causal, want_lse=True)
    assert kern == "flash_mfma_wide"
    assert not bool(out.isnan().any())
    rep = Hq // Hkv
    for b, h in ((0, 0), (B - 1, Hq - 1), (B // 2, Hq // 2 + 1)):
        hk = h // rep
        want, _ = O.sdpa_math(q[b:b + 1, h:h + 1], k[b:b + 1, hk:hk + 1], v[b:b + 1, hk:hk + 1], is_causal=causal, gemm="aten")
        assert max_abs(out[b:b + 1, h:h + 1], want) <= ABS_16BIT, (b, h)
        s = (q[b, h].double() @ k[b, hk].double().T) / math.sqrt(128)
        if causal:
            s = s.masked_fill(~torch.ones(Lq, Lk).tril().bool(), -math.inf)
        assert torch.allclose(lse[b, h].double().cpu(), torch.logsumexp(s, -1), rtol=0, atol=5e-4), (b, h)
    # the same call on inputs with padded rows and a transposed batch / head order
    qs = torch.empty(Hq, B, Lq, 160, dtype=dtype, device="cuda").permute(1, 0, 2, 3)[..., :128]
    ks = torch.empty(B, Hkv, Lk, 136, dtype=dtype, device="cuda")[..., :128]
    qs.copy_(qd); ks.copy_(kd)
    out2, _, _, kern2 = capi.sdpa(qs, ks, vd, is_causal=causal)
    assert kern2 == "flash_mfma_wide" and torch.equal(out2, out)


def test_config4_shape_slice_and_gqa_equivalence():
    """BASELINE config 4 (bf16 GQA decode B=64 Hq=32 Hkv=8 Lk=8192 D=128)."""
    B, Hq, Hkv, Lk = 64, 32, 8, 8192
    q = torch.randn(B, Hq, 1, 128).bfloat16()
    k, v = torch.randn(B, Hkv, Lk, 128).bfloat16(), torch.randn(B, Hkv, Lk, 128).bfloat16()
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    out, _, _, kern = capi.sdpa(qd, kd, vd)
    assert kern == "decode_split"
    want, _ = O.sdpa_math(q[:4], k[:4], v[:4], enable_gqa=True, gemm="aten")
    assert max_abs(out[:4], want) <= ABS_16BIT
    want, _ = O.sdpa_math(q[60:], k[60:], v[60:], enable_gqa=True, gemm="aten")
    assert max_abs(out[60:], want) <= ABS_16BIT
    # GQA by index mapping == explicit repeat_interleave of K/V (what the reference does)
    rep, _, _, _ = capi.sdpa(qd[:8], kd[:8].repeat_interleave(4, 1), vd[:8].repeat_interleave(4, 1))
    assert max_abs(out[:8], rep.cpu()) <= 4e-3
    ones, _, _, _ = capi.sdpa(qd, kd, torch.ones_like(vd))
    assert (ones.float() - 1).abs().max().item() <= 2 ** -7


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case_", [
    # B, Hq, Hkv, Lq, Lk, D, causal, mask
    (2, 4, 4, 200, 200, 80, True, None), (1, 8, 2, 130, 130, 96, False, None), (2, 2, 1, 77, 300, 40, False, "bool"),
    (1, 4, 4, 64, 64, 100, True, None), (2, 8, 2, 1, 900, 96, False, None), (1, 4, 1, 2, 700, 48, False, "add"),
    (1, 2, 2, 50, 50, 1, False, None), (1, 2, 2, 33, 65, 127, True, None),
    (2, 2, 2, 200, 200, 192, True, None), (1, 4, 2, 300, 500, 160, False, None), (1, 2, 2, 1, 700, 200, False, None),
    (1, 2, 1, 129, 257, 255, False, "bool"), (1, 2, 2, 70, 130, 129, False, "add")])
def test_head_sizes_between_the_mfma_kernels_are_padded_inside_the_library(case_, dtype):
    """16-bit head sizes below 256 other than 64 and 128, through the C ABI: the library copies q, k, v into
    its workspace with zero columns appended and runs the flash / decode kernels (prefill and decode
    shapes, GQA, causal, bool and additive masks, strided inputs)."""
    B, Hq, Hkv, Lq, Lk, D, causal, mk = case_
    torch.manual_seed(Lk + D)
    q = torch.randn(B, Lq, Hq, D).to(dtype).transpose(1, 2)            # heads and rows swapped in memory
    k, v = torch.randn(B, Hkv, Lk, D).to(dtype), torch.randn(B, Hkv, Lk, D).to(dtype)
    mask = None
    if mk == "bool":
        mask = torch.rand(B, 1, Lq, Lk) > 0.3
        mask[..., 0] = True
    elif mk == "add":
        mask = torch.randn(1, Hq, Lq, Lk).to(dtype)
    scale = O.round_to_dtype(1.0 / math.sqrt(D), dtype)
    out, _, lse, name = run(q, k, v, is_causal=causal, mask=mask, scale=scale, want_lse=True)
    want, _ = O.sdpa_math(q, k, v, is_causal=causal, attn_mask=mask, scale=scale, enable_gqa=True, gemm="aten")
    assert name == "padded_mfma" and out.shape == (B, Hq, Lq, D)
    assert max_abs(out, want) <= ABS_16BIT
    assert bool(torch.isfinite(lse).all())


# ---- the composed route: batched products + one row kernel, for large problems no fused kernel takes ----

def _composed_case(dtype, B, Hq, Hkv, Lq, Lk, D, Dv=None, **kw):
    Dv = Dv or D
    q, k, v = torch.randn(B, Hq, Lq, D).to(dtype), torch.randn(B, Hkv, Lk, D).to(dtype), torch.randn(B, Hkv, Lk, Dv).to(dtype)
    return q, k, v


def test_composed_route_fp32_causal_with_weights_and_lse():
    """fp32 at a size where the general kernel would take tens of milliseconds: the reference's
    composition run with the library's own products; outputs, weights and log-sum-exp."""
    torch.manual_seed(3)
    q, k, v = _composed_case(torch.float32, 2, 8, 8, 1024, 1024, 64)
    out, attn, lse, name = run(q, k, v, is_causal=True, want_attn=True, want_lse=True)
    assert name == "composed"
    want, wattn = O.sdpa_math(q, k, v, is_causal=True, gemm="aten")
    assert rel_err(out, want) <= REL_F32 and rel_err(attn, wattn) <= REL_F32
    assert float(attn.cpu().triu(1).abs().max()) == 0.0
    ref_lse = torch.logsumexp((q @ k.transpose(-1, -2) * 0.125).masked_fill(~torch.ones(1024, 1024).tril().bool(), -math.inf), -1)
    assert torch.allclose(lse.cpu(), ref_lse, rtol=1e-5, atol=1e-5)
    out2, _, _, _ = run(q, k, v, is_causal=True)              # scores in the workspace instead of the weights tensor
    assert torch.equal(out2.cpu(), out.cpu())


@pytest.mark.parametrize("cap", [None, 3 * 512 * 1024, 100 * 1024])
def test_composed_route_gqa_masks_and_pieces(cap, monkeypatch):
    """Grouped heads (the q heads of a kv head share its keys), a broadcast bool mask and an
    additive one, Lq != Lk, Dv != D; with the score bound lowered the same problem runs a few heads
    at a time and in blocks of query rows."""
    if cap is not None:
        monkeypatch.setenv("PARAS_SDPA_SCORE_CAP", str(cap))
    torch.manual_seed(4)
    q, k, v = _composed_case(torch.float32, 2, 8, 2, 512, 1024, 64, Dv=96)
    mask = torch.rand(2, 1, 512, 1024) > 0.3
    mask[0, 0, 7] = False                                     # a query that sees no key: NaN like the reference
    out, attn, _, name = run(q, k, v, mask=mask, want_attn=True)
    assert name == "composed"
    want, wattn = O.sdpa_math(q, k, v, attn_mask=mask, enable_gqa=True, gemm="aten")
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(out.cpu()), nan) and bool(nan[0, :, 7].all())
    assert rel_err(torch.nan_to_num(out.cpu()), torch.nan_to_num(want)) <= REL_F32
    assert rel_err(torch.nan_to_num(attn.cpu()), torch.nan_to_num(wattn)) <= REL_F32
    bias = torch.randn(1, 8, 512, 1024)
    out, _, _, name = run(q, k, v, mask=bias)
    assert name == "composed"
    want, _ = O.sdpa_math(q, k, v, attn_mask=bias, enable_gqa=True, gemm="aten")
    assert rel_err(out, want) <= REL_F32
    # one q head per kv head: several heads per piece
    q1, k1, v1 = _composed_case(torch.float32, 2, 6, 6, 640, 768, 80)
    out, _, _, name = run(q1, k1, v1, is_causal=True)
    assert name == "composed"
    want, _ = O.sdpa_math(q1, k1, v1, is_causal=True, gemm="aten")
    assert rel_err(out, want) <= REL_F32


def test_composed_route_fp64_and_wide_16_bit_heads():
    torch.manual_seed(5)
    q, k, v = _composed_case(torch.float64, 1, 4, 4, 2048, 2048, 32)
    out, _, _, name = run(q, k, v)
    assert name == "composed"
    want, _ = O.sdpa_math(q, k, v, gemm="aten")
    assert rel_err(out, want) <= 1e-12
    # bf16 with a head size no MFMA attention kernel has: the products still run on the matrix cores
    q, k, v = _composed_case(torch.bfloat16, 1, 4, 4, 1024, 1024, 256)
    out, attn, _, name = run(q, k, v, is_causal=True, want_attn=True)
    assert name == "composed"
    want, wattn = O.sdpa_math(q, k, v, is_causal=True, gemm="aten")
    assert max_abs(out, want) <= ABS_16BIT and max_abs(attn, wattn) <= ABS_16BIT
