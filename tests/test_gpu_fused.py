"""GPU parity of the fused RMSNorm / SwiGLU / rotate_half kernels, through the
C ABI, against the CPU oracle and the golden vectors.  Bar: bit-exact for
fp32 / bf16 / fp16 (the kernels evaluate the host engine's fp64 formula);
fp64 tensors within 1e-13 relative (summation order / exp last bit)."""
import pytest
import torch

import capi
import oracle as O
from conftest import assert_bit_exact
from golden_util import DTYPE_TAGS, case

pytestmark = pytest.mark.gpu
EXACT = [torch.float32, torch.bfloat16, torch.float16]


def dev(t):
    return t.cuda()


@pytest.mark.parametrize("tag", DTYPE_TAGS)
def test_golden_vectors(tag):
    c = case(f"rms_norm_{tag}")
    out, rstd = capi.rms_norm(dev(c["x"]), dev(c["w"]), 1e-6)
    assert_bit_exact(out, c["out"], "rms_norm")
    assert_bit_exact(rstd, c["rstd"], "rstd")
    gx, gw = capi.rms_norm_backward(dev(c["go"]), dev(c["x"]), dev(c["w"]), dev(c["rstd"]))
    assert_bit_exact(gx, c["gx"], "grad_input")
    if tag == "f32":
        assert torch.allclose(gw.cpu(), c["gw"], rtol=1e-6, atol=1e-6)   # slab-wise column sums
    else:
        assert_bit_exact(gw, c["gw"], "grad_weight")
    c = case(f"swiglu_{tag}")
    assert_bit_exact(capi.swiglu(dev(c["gate"]), dev(c["up"])), c["out"], "swiglu")
    gg, gu = capi.swiglu_backward(dev(c["go"]), dev(c["gate"]), dev(c["up"]))
    assert_bit_exact(gg, c["ggate"], "grad_gate")
    assert_bit_exact(gu, c["gup"], "grad_up")
    c = case(f"rotate_half_{tag}")
    assert_bit_exact(capi.rotate_half(dev(c["x"])), c["out"], "rotate_half")
    assert_bit_exact(capi.rotate_half(dev(c["x"]), True), c["bwd"], "rotate_half_backward")


@pytest.mark.parametrize("dtype", EXACT)
@pytest.mark.parametrize("shape", [(7, 200), (33, 4096), (5, 8192), (3, 10000), (64, 1024), (2, 8), (1, 1), (300, 264),
                                   (1000, 128), (37, 64), (515, 256), (77, 512), (9000, 1024), (5000, 2048), (40, 5120), (21, 2880),
                                   (6, 16384), (3, 12288), (1031, 32)])
def test_rms_norm_matches_oracle(dtype, shape):
    x = torch.randn(*shape).to(dtype)
    w = (1 + 0.02 * torch.randn(shape[1])).to(dtype)
    out, rstd = capi.rms_norm(dev(x), dev(w), 1e-6)
    want, wrstd = O.rms_norm(x, w, 1e-6)
    assert_bit_exact(out, want, f"rms_norm {dtype} {shape}")
    assert_bit_exact(rstd, wrstd, "rstd")


def test_rms_norm_unaligned_and_3d():
    base = torch.randn(4 * 6 * 40 + 3).bfloat16()
    x = base[3:].view(4, 6, 40)            # data pointer not 16-byte aligned on the device copy below
    w = torch.randn(40).bfloat16()
    xd = dev(base)[3:].view(4, 6, 40)
    out, rstd = capi.rms_norm(xd, dev(w), 1e-5)
    want, wrstd = O.rms_norm(x.contiguous(), w, 1e-5)
    assert_bit_exact(out, want, "unaligned rms_norm")
    assert out.shape == (4, 6, 40) and rstd.shape == (24,)


def test_rms_norm_fp64_and_empty():
    x, w = torch.randn(9, 300, dtype=torch.float64), torch.randn(300, dtype=torch.float64)
    out, rstd = capi.rms_norm(dev(x), dev(w), 1e-6)
    want, _ = O.rms_norm(x, w, 1e-6)
    assert torch.allclose(out.cpu(), want, rtol=1e-13, atol=1e-13)
    out, rstd = capi.rms_norm(torch.empty(0, 8, device="cuda"), torch.ones(8, device="cuda"), 1e-6)
    assert out.shape == (0, 8) and rstd.shape == (0,)


@pytest.mark.parametrize("dtype", EXACT)
@pytest.mark.parametrize("n", [1, 13, 4096, 100003])
def test_swiglu_matches_oracle(dtype, n):
    gate, up = (3 * torch.randn(n)).to(dtype), torch.randn(n).to(dtype)
    assert_bit_exact(capi.swiglu(dev(gate), dev(up)), O.swiglu(gate, up), f"swiglu {dtype} n={n}")


def test_swiglu_extreme_gates_take_the_exact_tier():
    """Gates outside the range of the fp32 fast path, zeros, infinities, NaN."""
    vals = [0.0, -0.0, 1e-30, -1e-30, -8.0, -8.5, -20.0, -60.0, -100.0, -700.0, 8.0, 60.0, 61.0, 100.0, 3e38,
            float("inf"), float("-inf"), float("nan")]
    gate = torch.tensor(vals).repeat_interleave(len(vals))
    up = torch.tensor(vals).repeat(len(vals))
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        g, u = gate.to(dtype), up.to(dtype)
        assert_bit_exact(capi.swiglu(dev(g), dev(u)), O.swiglu(g, u), f"swiglu extremes {dtype}")


def test_swiglu_every_bf16_gate():
    """All 65536 bf16 gate bit patterns against a few up values: the two-tier
    evaluation equals the fp64-then-round definition everywhere."""
    gate = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    for upv in (1.0, -0.3, 7.25, 1e-3):
        up = torch.full_like(gate, upv)
        assert_bit_exact(capi.swiglu(dev(gate), dev(up)), O.swiglu(gate, up), f"all gates, up={upv}")


@pytest.mark.parametrize("dtype", EXACT)
def test_backward_ops_match_oracle(dtype):
    x, w, go = torch.randn(50, 320).to(dtype), torch.randn(320).to(dtype), torch.randn(50, 320).to(dtype)
    _, rstd = O.rms_norm(x, w, 1e-6)
    gx, gw = capi.rms_norm_backward(dev(go), dev(x), dev(w), dev(rstd))
    wgx, wgw = O.rms_norm_backward(go, x, w, rstd)
    assert_bit_exact(gx, wgx, "rms_norm grad_input")
    if dtype == torch.float32:
        assert torch.allclose(gw.cpu(), wgw, rtol=1e-6, atol=1e-6)
    else:
        assert_bit_exact(gw, wgw, "rms_norm grad_weight")
    gate, up, g2 = torch.randn(1000).to(dtype), torch.randn(1000).to(dtype), torch.randn(1000).to(dtype)
    gg, gu = capi.swiglu_backward(dev(g2), dev(gate), dev(up))
    wgg, wgu = O.swiglu_backward(g2, gate, up)
    assert_bit_exact(gg, wgg, "swiglu grad_gate")
    assert_bit_exact(gu, wgu, "swiglu grad_up")
    xr = torch.randn(6, 10).to(dtype)
    assert_bit_exact(capi.rotate_half(dev(xr)), O.rotate_half(xr), "rotate_half")
    with pytest.raises(capi.ParasError):
        capi.rotate_half(torch.randn(4, 7, device="cuda"))          # odd last dim


def test_full_size_rms_norm_and_swiglu_bf16():
    """BASELINE config 2 at its real size, bit-exact against the oracle."""
    x = torch.randn(16384, 4096).bfloat16()
    w = (1 + 0.02 * torch.randn(4096)).bfloat16()
    out, rstd = capi.rms_norm(dev(x), dev(w), 1e-6)
    want, wrstd = O.rms_norm(x, w, 1e-6)
    assert_bit_exact(out, want, "rms_norm 16384x4096")
    assert_bit_exact(rstd, wrstd, "rstd")
    del x, out, want
    # SwiGLU: a 2048-row slab of the 16384 x 14336 tensor against the oracle,
    # the whole tensor through size-independent properties
    gate, up = torch.randn(16384, 14336).bfloat16(), torch.randn(16384, 14336).bfloat16()
    gd, ud = dev(gate), dev(up)
    res = capi.swiglu(gd, ud)
    assert_bit_exact(res[:2048], O.swiglu(gate[:2048], up[:2048]), "swiglu slab")
    assert_bit_exact(res[-64:], O.swiglu(gate[-64:], up[-64:]), "swiglu tail")
    neg = capi.swiglu(gd, -ud)
    assert torch.equal(neg.view(torch.int16) ^ res.view(torch.int16),
                       torch.full_like(res.view(torch.int16), -32768))    # odd in `up`, bit for bit


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(70, 4096), (33, 2048), (16, 520), (300, 1024), (5, 8), (37, 8192), (20, 5120), (9, 8200),
                                   (45, 6144), (50, 3072), (130, 1536), (70, 512), (31, 7168), (25, 2880),
                                   (1000, 128), (37, 64), (100, 96), (3, 256), (515, 512), (1, 128), (70000, 128),
                                   (6, 16384), (5, 12288), (300, 9216), (40, 16376)])
def test_rms_norm_backward_one_pass_kernel(shape, dtype):
    """Row sizes the one-pass backward kernels take (16-byte aligned rows: several rows per wave up
    to 512 elements, a vector per thread up to 8192, two with the column sums in LDS up to 16384),
    with slabs of rows that are full, ragged and single."""
    rows, H = shape
    torch.manual_seed(rows + H)
    x, w, go = torch.randn(rows, H).to(dtype), (1 + 0.1 * torch.randn(H)).to(dtype), torch.randn(rows, H).to(dtype)
    _, rstd = O.rms_norm(x, w, 1e-6)
    gx, gw = capi.rms_norm_backward(dev(go), dev(x), dev(w), dev(rstd))
    wgx, wgw = O.rms_norm_backward(go, x, w, rstd)
    assert_bit_exact(gx, wgx, "rms_norm grad_input")
    assert_bit_exact(gw, wgw, "rms_norm grad_weight")


def test_rms_norm_forward_and_backward_random_shapes():
    """Forty random (rows, H) pairs over every row-length path of both directions (several rows per
    wave, one workgroup per row, walking workgroups, one or two vectors per thread, the scalar
    kernels for rows that are not whole 16-byte vectors), both 16-bit dtypes: bit-exact."""
    gen = torch.Generator().manual_seed(2024)
    widths = [8, 24, 64, 120, 128, 136, 256, 384, 512, 520, 1000, 1024, 1536, 2048, 2880, 3072, 4096, 4104, 5120, 6144, 7168, 8192,
              8200, 9216, 12288, 16384, 16392, 20480, 100, 130, 4097]
    for trial in range(40):
        H = widths[int(torch.randint(len(widths), (1,), generator=gen))]
        rows = int(torch.randint(1, max(2, min(3000, 600000 // H)), (1,), generator=gen))
        dtype = (torch.bfloat16, torch.float16)[trial % 2]
        x = torch.randn(rows, H, generator=gen).to(dtype)
        w = (1 + 0.1 * torch.randn(H, generator=gen)).to(dtype)
        go = torch.randn(rows, H, generator=gen).to(dtype)
        out, rstd = capi.rms_norm(dev(x), dev(w), 1e-6)
        wout, wrstd = O.rms_norm(x, w, 1e-6)
        assert_bit_exact(out, wout, f"rms_norm out {rows}x{H} {dtype}")
        assert_bit_exact(rstd, wrstd, f"rms_norm rstd {rows}x{H} {dtype}")
        gx, gw = capi.rms_norm_backward(dev(go), dev(x), dev(w), dev(wrstd))
        wgx, wgw = O.rms_norm_backward(go, x, w, wrstd)
        assert_bit_exact(gx, wgx, f"rms_norm grad_input {rows}x{H} {dtype}")
        assert_bit_exact(gw, wgw, f"rms_norm grad_weight {rows}x{H} {dtype}")


def test_rms_norm_backward_many_rows_are_dealt_round_robin():
    """The one-pass kernel runs at most two workgroups per compute unit; with more rows than that
    times 16 every workgroup takes rows b, b + G, b + 2G, ...: row counts around the switch, with
    workgroups that get one row more than others."""
    for rows, H in ((16384 + 32 + 5, 264), (16383, 264), (16384, 520), (8192 + 7, 264), (4200, 5120), (9001, 3072), (4100, 8192), (4200, 8200), (2100, 12288)):
        torch.manual_seed(rows)
        x, w, go = torch.randn(rows, H).bfloat16(), (1 + 0.1 * torch.randn(H)).bfloat16(), torch.randn(rows, H).bfloat16()
        _, rstd = O.rms_norm(x, w, 1e-6)
        gx, gw = capi.rms_norm_backward(dev(go), dev(x), dev(w), dev(rstd))
        wgx, wgw = O.rms_norm_backward(go, x, w, rstd)
        assert_bit_exact(gx, wgx, f"rms_norm grad_input {rows}x{H}")
        assert_bit_exact(gw, wgw, f"rms_norm grad_weight {rows}x{H}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(8192, 4096), (8192 + 512, 4096), (8192 + 100, 4096), (16384, 2048), (16384 + 1024, 2048),
                                   (16384 + 24, 2048)])
def test_rms_norm_backward_team_workgroups(shape, dtype):
    """Rows of 4096 (2048) elements whose count is a multiple of 2 (4) per compute unit run in
    workgroups of 2 (4) teams that share one partial column sum; the row counts that do not divide
    evenly take the one-team workgroups."""
    rows, H = shape
    torch.manual_seed(rows)
    x, w, go = torch.randn(rows, H).to(dtype), (1 + 0.1 * torch.randn(H)).to(dtype), torch.randn(rows, H).to(dtype)
    _, rstd = O.rms_norm(x, w, 1e-6)
    gx, gw = capi.rms_norm_backward(dev(go), dev(x), dev(w), dev(rstd))
    wgx, wgw = O.rms_norm_backward(go, x, w, rstd)
    assert_bit_exact(gx, wgx, f"rms_norm grad_input {rows}x{H}")
    assert_bit_exact(gw, wgw, f"rms_norm grad_weight {rows}x{H}")


def test_rms_norm_backward_general_path_with_more_than_a_million_rows():
    """fp32 takes the three-kernel path, whose partial column sums are laid out one slab of 16 rows
    per workgroup along grid x: more than 65535 slabs (1,048,560 rows) must work."""
    rows, H = 16 * 65535 + 40, 8
    x, w, go = torch.randn(rows, H), 1 + 0.1 * torch.randn(H), torch.randn(rows, H)
    _, rstd = O.rms_norm(x, w, 1e-6)
    gx, gw = capi.rms_norm_backward(dev(go), dev(x), dev(w), dev(rstd))
    wgx, wgw = O.rms_norm_backward(go, x, w, rstd)
    assert_bit_exact(gx, wgx, "rms_norm grad_input")
    assert torch.allclose(gw.cpu(), wgw, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rms_norm_backward_adversarial_magnitudes(dtype):
    """The one-pass backward on rows built to break a shortcut in its arithmetic: products g*w and
    g*x far below / above the fp32 range (bf16), subnormal results, a huge rstd (eps = 0 on a tiny
    row), rows of zeros and signed zeros, grad_x terms that cancel almost completely, and NaN / inf
    entries.  Bit for bit against the oracle; NaNs compare as NaNs."""
    torch.manual_seed(23)
    rows, H = 48, 1024
    big = 1e30 if dtype == torch.bfloat16 else 3e4
    tiny = 1e-30 if dtype == torch.bfloat16 else 1e-6
    x, go = torch.randn(rows, H), torch.randn(rows, H)
    w = 1 + 0.1 * torch.randn(H)
    go[0] *= tiny; x[1] *= tiny; go[2] *= tiny; x[2] *= tiny          # underflowing products
    go[3] *= big; x[4] *= big                                         # overflowing products (fp32), finite in fp64
    go[5] = 0.0; go[6] = -0.0; x[7] = 0.0; x[8, ::2] = 0.0; go[8, 1::2] = -0.0
    go[9] = x[9] * 3.0                                                # grad_out parallel to x: the two terms cancel
    go[10] = x[10]
    go[11, 5] = float("nan"); x[12, 7] = float("inf"); go[13, 3] = float("-inf"); go[13, 4] = float("inf")
    x[14] *= 1e-3; x[15] *= 250.0
    w[17] = 0.0; w[18] = -0.0; w[19] = tiny; w[20] = 200.0
    x, go, w = x.to(dtype), go.to(dtype), w.to(dtype)
    for eps in (1e-6, 0.0):
        _, rstd = O.rms_norm(x, w, eps)
        gx, gw = capi.rms_norm_backward(dev(go), dev(x), dev(w), dev(rstd))
        wgx, wgw = O.rms_norm_backward(go, x, w, rstd)
        assert_bit_exact(gx, wgx, f"rms_norm grad_input eps={eps}")
        assert_bit_exact(gw, wgw, f"rms_norm grad_weight eps={eps}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rotate_half_vector_path_and_fallbacks(dtype):
    for shape in [(3, 5, 128), (7, 64), (2, 16), (4, 48), (3, 24), (5, 130)]:
        xr = torch.randn(*shape).to(dtype)
        assert_bit_exact(capi.rotate_half(dev(xr)), O.rotate_half(xr), f"rotate_half {shape}")
        assert_bit_exact(capi.rotate_half(dev(xr), True), O.rotate_half(xr, True), f"rotate_half backward {shape}")
    # a view that starts 2 bytes into an allocation: not 16-byte aligned
    buf = torch.randn(4 * 128 + 1).to(dtype)
    xr = buf[1:].view(4, 128)
    got = capi.rotate_half(dev(buf)[1:].view(4, 128))
    assert_bit_exact(got, O.rotate_half(xr.contiguous()), "rotate_half unaligned")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_swiglu_backward_every_gate_value(dtype):
    """The two-tier backward (fp32 with an error bound, fp64 next to rounding boundaries and around
    the zero of silu' at g = -1.278) against the oracle for every representable gate, with grad_out /
    up values of several magnitudes and signs, zeros included."""
    gate = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16).view(dtype)
    for dyv, uv in ((1.0, 1.0), (-0.3, 7.25), (1e-3, -2.5), (3.0, 0.0), (0.0, 1.0), (-250.0, 0.015625), (1.7, -1e-2)):
        dy, up = torch.full_like(gate, dyv), torch.full_like(gate, uv)
        gg, gu = capi.swiglu_backward(dev(dy), dev(gate), dev(up))
        wgg, wgu = O.swiglu_backward(dy, gate, up)
        for got, want, name in ((gg, wgg, "grad_gate"), (gu, wgu, "grad_up")):
            got = got.cpu()
            assert torch.equal(got.isnan(), want.isnan()), f"{name}: NaN positions, dy={dyv} up={uv}"
            keep = ~want.isnan()                       # (a NaN's sign and payload are not part of the contract)
            bad = int((got.view(torch.int16)[keep] != want.view(torch.int16)[keep]).sum())
            assert bad == 0, f"{name} for every gate, dy={dyv} up={uv}: {bad} elements differ bitwise"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_swiglu_backward_random_and_ragged(dtype):
    torch.manual_seed(17)
    for n, scale in ((8, 1.0), (1000003, 1.0), (4099, 6.0), (65536, 0.05)):
        gate, up, dy = (scale * torch.randn(n)).to(dtype), torch.randn(n).to(dtype), torch.randn(n).to(dtype)
        gg, gu = capi.swiglu_backward(dev(dy), dev(gate), dev(up))
        wgg, wgu = O.swiglu_backward(dy, gate, up)
        assert_bit_exact(gg, wgg, f"grad_gate n={n}")
        assert_bit_exact(gu, wgu, f"grad_up n={n}")
    # a view 2 bytes into its allocation: the element-wise kernel
    buf = torch.randn(3, 1025).to(dtype)
    g2, u2, d2 = buf[0, 1:], buf[1, 1:], buf[2, 1:]
    gg, gu = capi.swiglu_backward(dev(buf)[2, 1:], dev(buf)[0, 1:], dev(buf)[1, 1:])
    wgg, wgu = O.swiglu_backward(d2.contiguous(), g2.contiguous(), u2.contiguous())
    assert_bit_exact(gg, wgg, "grad_gate unaligned")
    assert_bit_exact(gu, wgu, "grad_up unaligned")


def assert_same_bits_nan_aware(got, want, what):
    """Bit for bit; a NaN must be a NaN at the same place.  bf16 NaNs also have the host's bits (its
    type writes every NaN as 0x7FC0); for the other types the sign of a NaN that an invalid operation
    produced is the host FPU's business (x86 makes it negative, the GPU positive) and is not compared."""
    got = got.cpu()
    assert got.shape == want.shape and got.dtype == want.dtype, what
    if want.dtype == torch.bfloat16:
        assert_bit_exact(got, want, what)
        return
    gn, wn = got.isnan(), want.isnan()
    assert torch.equal(gn, wn), f"{what}: NaNs at different places"
    it = {2: torch.int16, 4: torch.int32, 8: torch.int64}[want.element_size()]
    assert torch.equal(got.view(it)[~wn], want.view(it)[~wn]), f"{what}: bits differ"


SPECIALS = [0.0, -0.0, 1.5, -2.0, float("inf"), float("-inf"), float("nan"), 1e-30, -1e-30, 3e4, -3e4, 1e-7, 65504.0, 6e-8, -6e-8, 0.3]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_signed_zeros_infinities_and_nans_come_out_as_on_the_host(dtype):
    """RMSNorm forward and backward, SwiGLU forward and backward and rotate_half on rows that hold
    signed zeros, infinities, NaNs (also negative ones and ones with payloads), subnormal and huge
    values, weights that are zero or negative, eps = 0 on rows of zeros."""
    torch.manual_seed(3)
    H = 512
    x = torch.randn(16, H).to(dtype)
    for r, v in enumerate(SPECIALS):
        x[r, (r * 7) % H] = v
    x[1, ::2] = -0.0
    x[2] = 0.0
    x[3] = -0.0
    if dtype != torch.float32:
        x[9].view(torch.int16)[11] = 0x7FA5 if dtype == torch.bfloat16 else 0x7DA5
        x[10].view(torch.int16)[12] = -0x005B if dtype == torch.bfloat16 else -0x025B      # negative, with a payload
    w = (1 + 0.1 * torch.randn(H)).to(dtype)
    w[5], w[6], w[7] = -0.0, 0.0, -1.0
    for eps in (1e-6, 0.0):
        out, rstd = capi.rms_norm(dev(x), dev(w), eps)
        wo, wr = O.rms_norm(x, w, eps)
        assert_same_bits_nan_aware(out, wo, f"rms_norm {dtype} eps={eps}")
        assert_same_bits_nan_aware(rstd, wr, f"rstd {dtype} eps={eps}")
        if dtype != torch.float32:          # (fp32 column sums are compared with a tolerance elsewhere)
            go = torch.randn(16, H).to(dtype)
            go[0, 3], go[4, 9] = -0.0, float("nan")
            go[2] = -0.0
            gx, gw = capi.rms_norm_backward(dev(go), dev(x), dev(w), dev(wr))
            wgx, wgw = O.rms_norm_backward(go, x, w, wr)
            assert_same_bits_nan_aware(gx, wgx, f"rms_norm grad_x {dtype} eps={eps}")
            assert_same_bits_nan_aware(gw, wgw, f"rms_norm grad_w {dtype} eps={eps}")
    g = torch.tensor(SPECIALS).repeat(16, 1).to(dtype)
    u = torch.tensor(SPECIALS).view(16, 1).repeat(1, 16).to(dtype)
    assert_same_bits_nan_aware(capi.swiglu(dev(g), dev(u)), O.swiglu(g, u), f"swiglu {dtype}")
    go = torch.randn(16, 16).to(dtype)
    go[0], go[1], go[2, 3], go[3, 4] = -0.0, 0.0, float("nan"), float("inf")
    a, b = capi.swiglu_backward(dev(go), dev(g), dev(u))
    wa, wb = O.swiglu_backward(go, g, u)
    assert_same_bits_nan_aware(a, wa, f"swiglu grad_gate {dtype}")
    assert_same_bits_nan_aware(b, wb, f"swiglu grad_up {dtype}")
    xr = torch.tensor(SPECIALS).repeat(8, 8).to(dtype)
    if dtype != torch.float32:
        xr[0].view(torch.int16)[70] = 0x7FA5 if dtype == torch.bfloat16 else 0x7DA5        # a payload in each half
        xr[1].view(torch.int16)[5] = 0x7FA5 if dtype == torch.bfloat16 else 0x7DA5
    for backward in (False, True):
        got, want = capi.rotate_half(dev(xr), backward), O.rotate_half(xr, backward)
        if dtype == torch.bfloat16:
            assert_bit_exact(got, want, f"rotate_half {dtype} backward={backward}")
        else:
            assert_same_bits_nan_aware(got, want, f"rotate_half {dtype} backward={backward}")
