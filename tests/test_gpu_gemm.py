"""Dense NT GEMM (mm / bmm / addmm / linear on the device) through the C ABI.

The reference runs these on ATen-CPU with fp32 accumulation and one rounding
(csrc/ops/vision_ops.cpp:248-309,388-423); the oracle's matmul_nt accumulates
in double and rounds once.  Bar: every element within one 16-bit ulp of the
oracle (summation order is the only difference), and torch-CPU addmm / linear
as the library check for the epilogue.
"""
import math

import pytest
import torch

import capi
import oracle as O

pytestmark = pytest.mark.gpu


def ulp16(ref, dtype):
    mant = 7 if dtype == torch.bfloat16 else 10
    a = ref.double().abs().clamp_min(2.0 ** -14)
    return torch.exp2(torch.floor(torch.log2(a)) - mant)


def assert_gemm_close(out, ref, dtype):
    err = (out.double().cpu() - ref.double()).abs()
    tol = ulp16(ref, dtype) * 1.001 + 1e-6
    assert bool((err <= tol).all()), f"worst {err.max().item():.3e}, {(err > tol).sum().item()} beyond one ulp"


SHAPES = [(128, 256, 64), (1, 8, 64), (130, 257, 128), (300, 100, 192), (512, 1024, 1024), (77, 4096, 320),
          (4100, 2100, 64)]     # the last one: 256-row tiles with a single k-tile


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", SHAPES)
def test_gemm_nt_matches_oracle(shape, dtype):
    M, N, K = shape
    torch.manual_seed(M * 7 + N * 3 + K)
    a, b = torch.randn(M, K).to(dtype), (0.1 * torch.randn(N, K)).to(dtype)
    out = capi.gemm_nt(a.cuda(), b.cuda())
    assert_gemm_close(out, O.matmul_nt(a, b), dtype)


def test_gemm_nt_bias_and_addmm_epilogue():
    torch.manual_seed(1)
    M, N, K = 200, 384, 256
    dt = torch.bfloat16
    a, w, bias = torch.randn(M, K).to(dt), (0.05 * torch.randn(N, K)).to(dt), torch.randn(N).to(dt)
    out = capi.gemm_nt(a.cuda(), w.cuda(), bias.cuda())
    assert_gemm_close(out, torch.nn.functional.linear(a, w, bias), dt)        # library check: x W^T + b
    self_ = torch.randn(M, N).to(dt)
    out = capi.gemm_nt(a.cuda(), w.cuda(), self_.cuda(), alpha=0.5, beta=2.0)
    exact = 0.5 * (a.double() @ w.double().t()) + 2.0 * self_.double()
    assert_gemm_close(out, exact.to(dt), dt)
    assert_gemm_close(out, torch.addmm(self_, a, w.t(), beta=2.0, alpha=0.5), dt)


def test_gemm_nt_batched_strided_and_shared_operand():
    torch.manual_seed(2)
    B, M, N, K = 3, 96, 160, 128
    dt = torch.float16
    a = torch.randn(B, M, K + 8).to(dt)
    b = (0.1 * torch.randn(B, N, K)).to(dt)
    ad, bd = a.cuda()[:, :, :K], b.cuda()                           # rows 16-byte aligned, not dense
    a = a[:, :, :K]
    assert not ad.is_contiguous()
    out = capi.gemm_nt(ad, bd)
    for i in range(B):
        assert_gemm_close(out[i], O.matmul_nt(a[i].contiguous(), b[i]), dt)
    out = capi.gemm_nt(ad, bd[0])                                   # one weight matrix for the whole batch
    for i in range(B):
        assert_gemm_close(out[i], O.matmul_nt(a[i].contiguous(), b[0]), dt)


def test_gemm_nt_errors_and_empty():
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(capi.ParasError, match="leading dimension"):
        a = z(8, 64)
        capi.check(capi.lib().paras_gemm_nt(a.data_ptr(), a.data_ptr(), None, a.data_ptr(), 8, 8, 64, 32, 64, 8, 0, 1, 0, 0, 0, 0,
                                            1.0, 0.0, capi.BF16, capi._stream()))
    assert capi.gemm_nt(z(0, 64), z(8, 64)).shape == (0, 8)
    assert torch.equal(capi.gemm_nt(z(4, 0), z(8, 0)), z(4, 8))          # empty contraction: zeros


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16, torch.float16])
def test_gemm_nt_general_kernel(dtype):
    """What the MFMA kernels do not take -- fp32 / fp64 tensors, contraction sizes that are not a
    multiple of 64, rows that are not 16-byte aligned -- runs on the general device kernel."""
    torch.manual_seed(13)
    for (M, N, K) in [(1, 1, 1), (17, 9, 30), (70, 130, 65), (64, 64, 16), (129, 65, 200)]:
        a, b = torch.randn(M, K).to(dtype), (torch.randn(N, K) / math.sqrt(K)).to(dtype)
        got = capi.gemm_nt(a.cuda(), b.cuda())
        if dtype in (torch.bfloat16, torch.float16):
            assert_gemm_close(got, O.matmul_nt(a, b), dtype)
        else:
            want = a.double() @ b.double().t()
            tol = 1e-5 if dtype == torch.float32 else 1e-13
            assert torch.allclose(got.double().cpu(), want, rtol=tol, atol=tol)
        bias = torch.randn(N).to(dtype)
        got = capi.gemm_nt(a.cuda(), b.cuda(), bias.cuda(), alpha=0.5, beta=2.0)
        want = 0.5 * (a.double() @ b.double().t()) + 2.0 * bias.double()
        tol = {torch.float32: 1e-5, torch.float64: 1e-13}.get(dtype, 2e-2)
        assert torch.allclose(got.double().cpu(), want, rtol=tol, atol=tol)
    if dtype == torch.bfloat16:                                              # a multiple of 64, but rows 2 bytes off alignment
        buf = torch.randn(40 * 128 + 1).to(dtype).cuda()
        a = buf[1:].view(40, 128)
        b = (0.1 * torch.randn(24, 128)).to(dtype).cuda()
        assert_gemm_close(capi.gemm_nt(a, b), O.matmul_nt(a.cpu(), b.cpu()), dtype)


def test_gemm_nt_fp32_on_the_matrix_cores():
    """fp32 products with enough outputs for 128 x 128 tiles run on v_mfma_f32_32x32x2_f32 (full
    fp32 multiplies): ragged M, N, K, rows that are not 16-byte aligned (scalar staging), a batch
    with a shared weight, alpha / beta with a bias and with a full addend; 1e-5 against fp64."""
    torch.manual_seed(21)
    def close(got, want):
        scale = want.abs().max().item()
        assert (got.double().cpu() - want).abs().max().item() <= 1e-5 * scale
    for (M, N, K) in [(1024, 1024, 512), (1000, 777, 333), (130, 4100, 17), (4096, 640, 2048)]:
        a, b = torch.randn(M, K), torch.randn(N, K) / math.sqrt(K)
        close(capi.gemm_nt(a.cuda(), b.cuda()), a.double() @ b.double().t())
    a, b = torch.randn(700, 259), torch.randn(900, 259)                       # K odd: no 16-byte loads
    bias, full = torch.randn(900), torch.randn(700, 900)
    close(capi.gemm_nt(a.cuda(), b.cuda(), bias.cuda(), alpha=0.5, beta=2.0), 0.5 * (a.double() @ b.double().t()) + 2.0 * bias.double())
    close(capi.gemm_nt(a.cuda(), b.cuda(), full.cuda(), alpha=-1.25, beta=0.75), -1.25 * (a.double() @ b.double().t()) + 0.75 * full.double())
    buf = torch.randn(512 * 260 + 1).cuda()                                    # rows 4 bytes off 16-byte alignment
    av = buf[1:].view(512, 260)[:, :256]
    bw = torch.randn(640, 256)
    close(capi.gemm_nt(av, bw.cuda()), av.cpu().double() @ bw.double().t())
    a3, b2 = torch.randn(6, 300, 128), torch.randn(512, 128)                   # batched activations, one weight
    close(capi.gemm_nt(a3.cuda(), b2.cuda()), a3.double() @ b2.double().t())
    a3, b3 = torch.randn(5, 256, 96), torch.randn(5, 384, 96)                  # a weight per batch entry
    close(capi.gemm_nt(a3.cuda(), b3.cuda()), a3.double() @ b3.double().transpose(1, 2))


def test_gemm_nt_linearity_at_projection_size():
    """Size-independent property at a transformer projection shape: (2 a) W^T == 2 (a W^T) bit for
    bit, since scaling by a power of two commutes with every rounding; plus sampled rows vs the oracle."""
    torch.manual_seed(3)
    M, N, K = 4096, 4096, 4096
    dt = torch.bfloat16
    a1 = torch.randn(M, K, device="cuda").to(dt)
    a2 = a1 * 2                                                     # exact: a power of two
    w = (0.02 * torch.randn(N, K, device="cuda")).to(dt)
    y1, y2 = capi.gemm_nt(a1, w), capi.gemm_nt(a2, w)
    assert torch.equal(y2, y1 * 2)                                  # scaling by 2 commutes with every rounding
    rows = torch.randint(0, M, (8,))
    ref = O.matmul_nt(a1[rows].cpu(), w.cpu())
    assert_gemm_close(y1[rows], ref, dt)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gemm_nt_many_tiles_with_ragged_edges(dtype):
    """Thousands of tiles, with M and N that are not multiples of the tile; sampled rows (first,
    last, tile boundaries) against the oracle."""
    torch.manual_seed(9)
    M, N, K = 8269, 4129, 192
    a = torch.randn(M, K, device="cuda").to(dtype)
    b = (0.1 * torch.randn(N, K, device="cuda")).to(dtype)
    bias = torch.randn(N, device="cuda").to(dtype)
    out = capi.gemm_nt(a, b)
    rows = torch.tensor([0, 1, 127, 128, 255, 256, 257, 4095, 4096, 8191, 8192, M - 2, M - 1])
    ref = O.matmul_nt(a[rows].cpu(), b.cpu())
    assert_gemm_close(out[rows], ref, dtype)
    out2 = capi.gemm_nt(a, b, bias, alpha=1.0, beta=1.0)
    assert_gemm_close(out2[rows], torch.nn.functional.linear(a[rows].cpu(), b.cpu(), bias.cpu()), dtype)
    # whole-matrix property: doubling A doubles every output bit for bit (away from f16's subnormals,
    # where 2 * round(v) and round(2 v) keep different numbers of bits)
    big = out.float().abs() > 1e-3
    assert torch.equal(capi.gemm_nt(a * 2, b)[big], (out * 2)[big])


_EIGHT_WAVES_CHILD = r"""
import hashlib, sys, torch
sys.path.insert(0, sys.argv[1])
import capi
torch.manual_seed(33)
a = torch.randn(4, 2100, 128).bfloat16().cuda()
b = (0.1 * torch.randn(4, 2100, 128)).bfloat16().cuda()
out = capi.gemm_nt(a, b)
T, E, k, H, I = 4096, 2, 2, 1024, 512
logits, x = torch.randn(T, E).bfloat16().cuda(), torch.randn(T, H).bfloat16().cuda()
wg, wu = (0.03 * torch.randn(E, I, H)).bfloat16().cuda(), (0.03 * torch.randn(E, I, H)).bfloat16().cuda()
wd = (0.03 * torch.randn(E, H, I)).bfloat16().cuda()
topi, topw, order, inv, counts, offsets = capi.moe_route(logits, k)
y = capi.moe_ffn(x, wg, wu, wd, topw, order, inv, offsets, k)
for t in (out, y):
    print(hashlib.sha256(t.cpu().view(torch.int16).numpy().tobytes()).hexdigest())
"""


def test_256_row_tiles_on_eight_waves_give_the_same_bits():
    """PARAS_GEMM_EIGHT_WAVES=1 (read once per process, hence the child process) sends the 256-row tiles of the
    dense product and of the expert FFN to the eight-wave kernels on 32 x 32 x 16 MFMAs.  They add the same
    products in the same order as the four-wave kernels on 16 x 16 x 32: identical outputs, compared by digest."""
    import os, subprocess, sys
    here = os.path.dirname(os.path.abspath(__file__))
    def run(extra):
        env = {k: v for k, v in os.environ.items() if k != "PARAS_GEMM_EIGHT_WAVES"}
        env.update(extra)
        r = subprocess.run([sys.executable, "-c", _EIGHT_WAVES_CHILD, here], env=env, capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        return r.stdout.split()
    four, eight = run({}), run({"PARAS_GEMM_EIGHT_WAVES": "1"})
    assert len(four) == 2 and four == eight


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(4352, 4096, 256), (700, 512, 128), (64, 1024, 512), (8, 512, 256)])
def test_gemm_nt_nan_and_infinity_go_where_ieee_sends_them(shape, dtype):
    """A NaN in one row of A, an infinity in one row of B, on every tile form (256-row, 128-row, the
    split contraction of few rows, the weight-streaming kernel): NaNs exactly where fp32 arithmetic
    puts them (that row, that column; in bfloat16 with the host's NaN encoding), infinities with their signs,
    everything else as without them."""
    M, N, K = shape
    torch.manual_seed(M)
    a = torch.randn(M, K).to(dtype)
    b = (0.1 * torch.randn(N, K)).to(dtype)
    clean = capi.gemm_nt(a.cuda(), b.cuda()).cpu()
    a[M // 3, 5] = float("nan")
    b[N // 2, 7] = float("inf")
    got = capi.gemm_nt(a.cuda(), b.cuda()).cpu()
    ref = (a.float() @ b.float().T).to(dtype)
    assert torch.equal(got.isnan(), ref.isnan()) and torch.equal(got.isinf(), ref.isinf())
    assert bool(got[M // 3].isnan().all()) and bool(got[:, N // 2].isinf().sum() >= M - 2)
    assert torch.equal(got[got.isinf()], ref[ref.isinf()])
    if dtype == torch.bfloat16:
        # one NaN encoding in bfloat16, the oracle's; float16 keeps the sign of the fp32 NaN, and which sign
        # a NaN sum gets is the adder's choice (the matrix cores and a CPU differ), so only bf16 is held to bits
        want_row = O.matmul_nt(a[M // 3: M // 3 + 1], b)
        assert torch.equal(got[M // 3: M // 3 + 1].view(torch.int16), want_row.view(torch.int16))
    keep = torch.ones(M, N, dtype=torch.bool)
    keep[M // 3] = False
    keep[:, N // 2] = False
    assert torch.equal(got[keep], clean[keep])


def test_gemm_nt_256_row_tiles_agree_with_128_row_tiles():
    """A batch of four problems is big enough for the 256-row tiles, each problem alone is not:
    both forms add the same products in the same order, so they agree bit for bit (ragged M and
    N, strided batch)."""
    torch.manual_seed(21)
    Bt, M, N, K = 4, 2100, 2100, 128      # 81 tiles of 256 x 256 each (-> 128 x 128 tiles), 324 together (-> 256-row tiles)
    a = torch.randn(Bt, M, K, device="cuda").bfloat16()
    b = (0.1 * torch.randn(Bt, N, K, device="cuda")).bfloat16()
    whole = capi.gemm_nt(a, b)
    assert whole.shape == (Bt, M, N)
    for i in range(Bt):
        assert torch.equal(whole[i], capi.gemm_nt(a[i], b[i])), f"batch {i}"
    ref = O.matmul_nt(a[3, -3:].cpu(), b[3].cpu())
    assert_gemm_close(whole[3, -3:], ref, torch.bfloat16)


@pytest.mark.parametrize("shape", [(2, 1100, 2100, 64), (1, 1024, 2048, 128), (3, 2300, 4200, 64), (1, 16384, 4096, 64)])
def test_gemm_nt_tiles_dealt_to_the_dies_in_blocks_cover_every_element(shape):
    """From 4 x 8 tiles of 256 x 256 on, the workgroups take their tiles in blocks of 4 x 8 per die,
    on a grid padded to whole blocks and to eight blocks at a time: every element of every batch
    entry has to come out, none twice from a wrong tile.  Whole matrix against the oracle (which
    fits here: one k-tile or two)."""
    Bt, M, N, K = shape
    torch.manual_seed(33)
    a = torch.randn(Bt, M, K, device="cuda").bfloat16()
    b = (0.1 * torch.randn(Bt, N, K, device="cuda")).bfloat16()
    out = capi.gemm_nt(a, b)
    assert out.shape == (Bt, M, N)
    for i in range(Bt):
        assert_gemm_close(out[i], O.matmul_nt(a[i].cpu(), b[i].cpu()), torch.bfloat16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 4096, 4096), (16, 100, 64), (17, 1027, 320), (64, 4096, 1024), (100, 515, 192),
                                   (128, 2050, 4096)])
def test_gemm_nt_few_rows(shape, dtype):
    """M <= 128 (decode-time projections) runs on the weight-streaming kernel: plain product,
    bias + scaled addend, N with and without 8-byte aligned output rows."""
    M, N, K = shape
    torch.manual_seed(M + N + K)
    a = torch.randn(M, K).to(dtype)
    b = (torch.randn(N, K) / math.sqrt(K)).to(dtype)
    assert_gemm_close(capi.gemm_nt(a.cuda(), b.cuda()), O.matmul_nt(a, b), dtype)
    bias = torch.randn(N).to(dtype)
    got = capi.gemm_nt(a.cuda(), b.cuda(), bias.cuda(), alpha=1.0, beta=1.0)
    assert_gemm_close(got, torch.nn.functional.linear(a, b, bias), dtype)
    addm = torch.randn(M, N).to(dtype)
    got = capi.gemm_nt(a.cuda(), b.cuda(), addm.cuda(), alpha=0.5, beta=2.0)
    want = torch.addmm(addm.float(), a.float(), b.float().t(), beta=2.0, alpha=0.5)
    err = (got.float().cpu() - want).abs()
    assert bool((err <= 2 * ulp16(want, dtype) + 1e-6).all())


def test_gemm_nt_few_rows_batched():
    torch.manual_seed(8)
    a = torch.randn(6, 40, 256, device="cuda").bfloat16()
    b = (0.1 * torch.randn(6, 72, 256, device="cuda")).bfloat16()
    out = capi.gemm_nt(a, b)
    for i in range(6):
        assert_gemm_close(out[i], O.matmul_nt(a[i].cpu(), b[i].cpu()), torch.bfloat16)
    shared = capi.gemm_nt(a, b[0])                      # one weight matrix for the whole batch
    for i in range(6):
        assert torch.equal(shared[i], capi.gemm_nt(a[i], b[0]))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(32, 4096, 4096), (64, 4096, 1024), (64, 1027, 4096), (100, 1536, 2048), (128, 2050, 4096),
                                   (33, 640, 1088), (48, 4096, 2048), (49, 384, 4096), (128, 4096, 14336), (77, 130, 704)])
def test_gemm_nt_few_rows_with_workspace(shape, dtype):
    """32 to 128 rows with the workspace the library asks for: the contraction is split over
    workgroups (of the few-row kernel up to 48 rows, of the 128 x 128 tile kernel above) and the
    partial sums are added in a fixed order -- same bar as every other GEMM kernel, same result on
    every call, with bias / scaled addend and ragged N and K splits."""
    M, N, K = shape
    torch.manual_seed(M + N + K)
    a = torch.randn(M, K).to(dtype)
    b = (torch.randn(N, K) / math.sqrt(K)).to(dtype)
    assert capi.lib().paras_gemm_nt_workspace(M, N, K, 1, capi.DT[dtype]) > 0
    got = capi.gemm_nt(a.cuda(), b.cuda(), workspace=True)
    assert_gemm_close(got, O.matmul_nt(a, b), dtype)
    assert torch.equal(got, capi.gemm_nt(a.cuda(), b.cuda(), workspace=True))          # deterministic
    bias = torch.randn(N).to(dtype)
    got = capi.gemm_nt(a.cuda(), b.cuda(), bias.cuda(), alpha=1.0, beta=1.0, workspace=True)
    assert_gemm_close(got, torch.nn.functional.linear(a, b, bias), dtype)
    addm = torch.randn(M, N).to(dtype)
    got = capi.gemm_nt(a.cuda(), b.cuda(), addm.cuda(), alpha=0.5, beta=2.0, workspace=True)
    want = torch.addmm(addm.float(), a.float(), b.float().t(), beta=2.0, alpha=0.5)
    assert bool(((got.float().cpu() - want).abs() <= 2 * ulp16(want, dtype) + 1e-6).all())


def test_gemm_nt_few_rows_and_many_columns_take_the_tile_kernel():
    """33 to 128 rows against a vocabulary-sized weight matrix: enough 128 x 128 tiles to fill the
    chip, so no workspace is asked for and the result is the tile kernel's."""
    torch.manual_seed(44)
    M, N, K = 100, 24576 + 70, 256
    a = torch.randn(M, K).bfloat16()
    b = (torch.randn(N, K) / 16).bfloat16()
    assert capi.lib().paras_gemm_nt_workspace(M, N, K, 1, capi.BF16) == 0
    got = capi.gemm_nt(a.cuda(), b.cuda(), workspace=True)
    assert_gemm_close(got, O.matmul_nt(a, b), torch.bfloat16)
    bias = torch.randn(N).bfloat16()
    got = capi.gemm_nt(a.cuda(), b.cuda(), bias.cuda(), alpha=1.0, beta=1.0)
    assert_gemm_close(got, torch.nn.functional.linear(a, b, bias), torch.bfloat16)
    # batched: 3 x 64 tiles
    a3 = torch.randn(3, 60, 256, device="cuda").bfloat16()
    b3 = (torch.randn(3, 8192, 256, device="cuda") / 16).bfloat16()
    out = capi.gemm_nt(a3, b3, workspace=True)
    for i in range(3):
        assert_gemm_close(out[i], O.matmul_nt(a3[i].cpu(), b3[i].cpu()), torch.bfloat16)


def test_gemm_nt_workspace_batched_and_shapes_that_need_none():
    torch.manual_seed(6)
    a = torch.randn(3, 48, 1024, device="cuda").bfloat16()
    b = (0.05 * torch.randn(3, 768, 1024, device="cuda")).bfloat16()
    out = capi.gemm_nt(a, b, workspace=True)
    for i in range(3):
        assert_gemm_close(out[i], O.matmul_nt(a[i].cpu(), b[i].cpu()), torch.bfloat16)
    L = capi.lib()
    assert L.paras_gemm_nt_workspace(8, 4096, 4096, 1, capi.BF16) == 0        # up to 16 rows: nothing to share
    assert L.paras_gemm_nt_workspace(4096, 4096, 4096, 1, capi.BF16) == 0     # tile kernels
    assert L.paras_gemm_nt_workspace(64, 4096, 4096, 1, capi.F32) == 0        # general kernel
    x = torch.randn(8, 256, device="cuda").bfloat16()
    w = torch.randn(64, 256, device="cuda").bfloat16()
    assert torch.equal(capi.gemm_nt(x, w, workspace=True), capi.gemm_nt(x, w))


def test_mfma_rate_probe_reports_a_plausible_rate():
    """The measurement aid bench.py prints beside the attention figure: a register-only MFMA loop
    cannot beat the published peak and, on a healthy MI355X, does not fall below a fifth of it."""
    import ctypes as C
    rate = C.c_double(0.0)
    capi.check(capi.lib().paras_mfma_rate_probe(1, 0, C.byref(rate)))
    assert 500.0 < rate.value < 2600.0
    assert capi.lib().paras_mfma_rate_probe(3, 0, C.byref(rate)) != 0          # only one or two wavefronts per SIMD
    assert b"wavefronts per SIMD" in capi.lib().paras_last_error()


def test_l2_stream_probe_reports_plausible_rates():
    """The streaming probe: regions that stay in L2 come in faster than regions that do not, and
    both at a rate a CU can plausibly reach (a GEMM tile of 256 x 256 needs about 40 B/ns per CU)."""
    import ctypes as C
    rate = C.c_double(0.0)
    got = {}
    for to_lds, kib in ((1, 64), (1, 512), (0, 64)):
        capi.check(capi.lib().paras_l2_stream_probe(to_lds, kib, C.byref(rate)))
        got[(to_lds, kib)] = rate.value
    assert 40.0 < got[(1, 64)] < 400.0, got            # measured 116 - 128 B/ns per CU
    assert 5.0 < got[(1, 512)] < got[(1, 64)], got      # measured 21 - 26 B/ns per CU from the last-level cache
    assert 10.0 < got[(0, 64)] < 400.0, got             # measured 33 B/ns per CU with eight loads in flight per wavefront
    assert capi.lib().paras_l2_stream_probe(1, 48, C.byref(rate)) != 0        # not a power of two


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(16384, 8, 4096), (5000, 1, 256), (3001, 17, 512), (2048, 32, 1024), (3001, 33, 512), (2048, 128, 1024), (700, 100, 192), (9000, 64, 4096)])
def test_gemm_nt_few_columns_and_many_rows(shape, dtype):
    """A router's logits and the like (tokens x experts): the few-row kernels with the operands in each
    other's place and the results stored transposed; plain, with a bias over the columns, with a full
    addend and a scale, and batched."""
    M, N, K = shape
    torch.manual_seed(M + N)
    a = torch.randn(M, K).to(dtype)
    b = (0.1 * torch.randn(N, K)).to(dtype)
    rows = torch.tensor([0, 1, 15, 16, 127, 128, M // 2, M - 2, M - 1])
    out = capi.gemm_nt(a.cuda(), b.cuda())
    assert out.shape == (M, N)
    assert_gemm_close(out[rows], O.matmul_nt(a[rows], b), dtype)
    # every element against an fp32 product on the device (nothing left unwritten, nothing misplaced;
    # that product sums in another order, so small results get an absolute allowance)
    ref = (a.cuda().float() @ b.cuda().float().t())
    assert bool(((out.float() - ref).abs() <= 2.0 ** -7 * ref.abs().clamp_min(0.05)).all())
    bias = torch.randn(N).to(dtype)
    out2 = capi.gemm_nt(a.cuda(), b.cuda(), bias.cuda())
    assert_gemm_close(out2[rows], torch.nn.functional.linear(a[rows], b, bias), dtype)
    full = torch.randn(M, N).to(dtype)
    out3 = capi.gemm_nt(a.cuda(), b.cuda(), full.cuda(), alpha=0.5, beta=2.0)
    want3 = (0.5 * (a[rows].double() @ b.double().t()) + 2.0 * full[rows].double())
    assert_gemm_close(out3[rows], want3, dtype)
    ab = torch.stack([a[:600], a[600:1200]]) if M >= 1200 else None
    if ab is not None:
        bb = torch.stack([b, b.flip(0)])
        ob = capi.gemm_nt(ab.cuda(), bb.cuda())
        for i in range(2):
            assert_gemm_close(ob[i, -3:], O.matmul_nt(ab[i, -3:], bb[i]), dtype)
