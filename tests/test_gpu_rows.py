"""Row softmax and row top-k on the device through the C ABI, against the oracle
(reference arithmetic: csrc/ops/pointwise_ops.cpp:926-981, 1292-1381) and the
reference tests' own checks (torch-CPU parity, tests/test_pointwise_ops.py:224-267,
369-413, including its tie literal)."""
import pytest
import torch

import capi
import oracle as O
from conftest import assert_bit_exact

pytestmark = pytest.mark.gpu
FLOATS = [torch.float32, torch.bfloat16, torch.float16, torch.float64]


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("shape", [(1, 1), (7, 8), (33, 300), (4, 5000), (2, 3, 129), (1001, 64), (37, 65), (10, 256), (3, 257), (5, 1024), (3, 1025), (2, 4096), (2, 4097)])
def test_softmax_matches_oracle(dtype, shape):
    torch.manual_seed(sum(shape))
    x = (3 * torch.randn(*shape)).to(dtype)
    got = capi.softmax_rows(x.cuda()).cpu()
    want = O.softmax_last(x)
    # device exp() and the host's libm may differ in the last bit of a double, and the row sum is
    # taken in a different order: after narrowing that shows, rarely, as one unit in the last place
    if dtype in (torch.bfloat16, torch.float16):
        diff = (got.view(torch.int16).int() - want.view(torch.int16).int()).abs()
        assert int(diff.max()) <= 1 and float((diff > 0).float().mean()) <= 1e-3
    else:
        assert torch.allclose(got, want, rtol=1e-6 if dtype == torch.float32 else 1e-13, atol=0)
    assert torch.allclose(got.double().sum(-1), torch.ones(shape[:-1], dtype=torch.float64), atol=2e-2 if dtype in (torch.bfloat16, torch.float16) else 1e-5)


def test_softmax_half_to_float_and_extremes():
    x = torch.tensor([[0.0, -1e4, 1e4, 5.0], [float("-inf"), 0.0, 0.0, float("-inf")]], dtype=torch.float16)
    got = capi.softmax_rows(x.cuda(), torch.float32).cpu()
    assert got.dtype == torch.float32
    assert torch.allclose(got, O.softmax_last(x, torch.float32), rtol=1e-6, atol=0)
    assert torch.allclose(got, torch.softmax(x.float(), -1), rtol=1e-6, atol=1e-30)
    with pytest.raises(capi.ParasError):
        capi.softmax_rows(torch.zeros(2, 4, device="cuda"), torch.float16)
    assert capi.softmax_rows(torch.zeros(0, 4, device="cuda")).shape == (0, 4)


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("largest", [True, False])
def test_topk_matches_oracle_bitwise(dtype, largest):
    torch.manual_seed(11)
    for shape, k in (((5, 8), 2), ((9, 64), 8), ((3, 1000), 17), ((2, 2, 300), 300), ((4, 7), 0), ((1001, 64), 2),
                     ((37, 65), 65), ((10, 256), 5), ((3, 257), 4)):
        x = torch.randn(*shape).to(dtype)
        x = (x * 4).round() / 4 if dtype != torch.float64 else x          # quantised: plenty of ties
        gv, gi = capi.topk_rows(x.cuda(), k, largest)
        wv, wi = O.topk_last(x, k, largest)
        assert_bit_exact(gi, wi, f"topk indices {shape} k={k}")
        assert_bit_exact(gv, wv, f"topk values {shape} k={k}")


def test_topk_reference_tie_literal_and_torch_parity():
    x = torch.tensor([[5.0, 3.0, 5.0, 5.0, 1.0, 3.0]])                  # tests/test_pointwise_ops.py:405-413
    v, i = capi.topk_rows(x.cuda(), 4)
    assert i.cpu().tolist() == [[0, 2, 3, 1]] and v.cpu().tolist() == [[5.0, 5.0, 5.0, 3.0]]
    torch.manual_seed(5)
    y = torch.randn(16, 257)                                              # distinct values: order is unique
    v, i = capi.topk_rows(y.cuda(), 9)
    tv, ti = torch.topk(y, 9, dim=-1)
    assert torch.equal(i.cpu(), ti) and torch.equal(v.cpu(), tv)
    with pytest.raises(capi.ParasError, match="k out of range"):
        capi.topk_rows(y.cuda(), 300)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("n", [264, 1024, 2048, 2056, 4096, 4104, 8192, 8200, 32768])
def test_softmax_rows_in_whole_16_byte_pieces(dtype, n):
    """Row lengths that are a multiple of eight (the kernel with 16-byte loads and stores), with the rows
    the host treats specially among ordinary ones: a NaN in the row, a row of NaNs, +inf and -inf
    in a row, a row of -inf, a constant row, a row with a spread of 200 (most weights underflow)."""
    torch.manual_seed(n)
    x = (3 * torch.randn(9, n)).to(dtype)
    nan, inf = float("nan"), float("inf")
    x[1, n // 2] = nan
    x[2] = nan
    x[3, 7], x[3, n - 1] = inf, -inf
    x[4] = -inf
    x[5] = 1.5
    x[6] = (torch.linspace(-100, 100, n)).to(dtype)
    x[7, 0] = -inf
    got, want = capi.softmax_rows(x.cuda()).cpu(), O.softmax_last(x)
    assert torch.equal(got.isnan(), want.isnan())
    bits = torch.int32 if dtype == torch.float32 else torch.int16
    if dtype == torch.float32:
        assert torch.allclose(got, want, rtol=1e-6, atol=0, equal_nan=True)
    else:
        diff = (got.view(bits).int() - want.view(bits).int()).abs()[~want.isnan()]
        assert int(diff.max()) <= 1 and float((diff > 0).float().mean()) <= 1e-3
        assert torch.equal(got.view(bits)[want.isnan()], want.view(bits)[want.isnan()])      # the host's NaN encoding
    assert torch.equal(got[5], want[5]) and bool((got[7, 0] == 0).item())
    # a view at an odd offset takes the element-wise kernel: same values
    buf = torch.zeros(9 * n + 1, dtype=dtype, device="cuda")
    buf[1:] = x.cuda().flatten()
    other = capi.softmax_rows(buf[1:].view(9, n)).cpu()
    if dtype == torch.float32:
        assert torch.allclose(other, got, rtol=1e-6, atol=0, equal_nan=True)       # (another order of the row's sum)
    else:
        odiff = (other.view(bits).int() - got.view(bits).int()).abs()[~want.isnan()]
        assert int(odiff.max()) <= 1 and float((odiff > 0).float().mean()) <= 1e-3


def test_short_rows_with_nan_and_infinities():
    """The one-wave-per-row kernels keep the host engine's conventions: a NaN never becomes the
    row maximum of a softmax; a top-k slot with no candidate reports index -1 and value 0."""
    x = torch.tensor([[1.0, float("nan"), 3.0, 2.0], [float("nan")] * 4, [float("inf"), 1.0, float("-inf"), 0.5]])
    got, want = capi.softmax_rows(x.cuda()).cpu(), O.softmax_last(x)
    assert torch.equal(got.isnan(), want.isnan())
    assert torch.allclose(got.nan_to_num(7.0), want.nan_to_num(7.0), rtol=1e-6, atol=0)
    gv, gi = capi.topk_rows(x.cuda(), 3)
    wv, wi = O.topk_last(x, 3)
    assert_bit_exact(gi, wi, "topk indices with NaN rows")
    assert torch.equal(gv.cpu().isnan(), wv.isnan()) and torch.equal(gv.cpu().nan_to_num(7.0), wv.nan_to_num(7.0))


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("n", [40, 200, 700])
def test_topk_rows_with_nans_follow_the_host_scan(dtype, n):
    """The host picks each slot by a scan from the left in which a NaN never replaces the running
    best and is never 'after' the previous slot: a NaN is chosen only as x[0] in slot 0, the slot
    after that has no candidate (index -1, value 0), and the one after that goes on from (0, -1).
    NaNs first, last, in runs and next to infinities, on the one-wave and the workgroup kernels,
    largest and smallest."""
    torch.manual_seed(n)
    x = torch.randn(12, n).to(dtype)
    nan, inf = float("nan"), float("inf")
    x[0, 5] = nan
    x[1, 0] = nan
    x[2, 0], x[2, 9] = nan, nan
    x[3, n - 1] = nan
    x[4, 1:5] = nan
    x[5, 0], x[5, 1] = nan, inf
    x[6, 0], x[6, 3] = inf, nan
    x[7, 0], x[7, 2], x[7, 3] = nan, 0.0, -0.0
    x[8, ::2] = nan
    x[9, 0], x[9, 1:] = 1.0, nan
    for k in (1, 3, min(n, 40)):
        for largest in (True, False):
            gv, gi = capi.topk_rows(x.cuda(), k, largest)
            wv, wi = O.topk_last(x, k, largest)
            assert_bit_exact(gi, wi, f"topk indices {dtype} n={n} k={k} largest={largest}")
            if dtype == torch.bfloat16 or not bool(wv.isnan().any()):
                assert_bit_exact(gv, wv, f"topk values {dtype} n={n} k={k} largest={largest}")
            else:
                assert torch.equal(gv.cpu().isnan(), wv.isnan()) and torch.equal(gv.cpu().nan_to_num(7.0), wv.nan_to_num(7.0))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("largest", [True, False])
def test_topk_long_rows_keep_one_candidate_per_thread(dtype, largest):
    """Vocabulary-sized rows run on the kernel that keeps one candidate per thread and refreshes only
    the one that was taken: quantised values (thousands of ties, signed zeros), k up to a few
    hundred, rows with NaNs, and rows with fewer eligible elements than k, where the host reports
    (0, -1) and goes on from there."""
    torch.manual_seed(91)
    for (rows, n), k in (((3, 9000), 50), ((2, 20000), 300), ((1, 128256), 50), ((4, 300), 300), ((2, 8192), 64), ((2, 8200), 7)):
        x = ((torch.randn(rows, n) * 4).round() / 4).to(dtype)
        x[0, 17] = -0.0
        x[0, 3] = 0.0
        if rows > 1:
            x[1, 5::3] = float("nan")
            x[1, 1] = float("inf")
        gv, gi = capi.topk_rows(x.cuda(), k, largest)
        wv, wi = O.topk_last(x, k, largest)
        assert_bit_exact(gi, wi, f"topk indices {(rows, n)} k={k}")
        assert_bit_exact(gv, wv, f"topk values {(rows, n)} k={k}")
    # fewer eligible elements than k; a NaN first; everything NaN but the first
    x = torch.randn(5, 600).to(dtype)
    x[0, 10:] = float("nan")
    x[1, 0] = float("nan")
    x[2, 1:] = float("nan")
    x[3, :] = float("nan")
    x[4, ::2] = float("nan")
    x[4, 1] = 0.0
    for k in (5, 40, 600):
        gv, gi = capi.topk_rows(x.cuda(), k, largest)
        wv, wi = O.topk_last(x, k, largest)
        assert_bit_exact(gi, wi, f"topk indices with few eligible elements k={k}")
        assert torch.equal(gv.cpu().isnan(), wv.isnan()) and torch.equal(gv.cpu().nan_to_num(7.0), wv.nan_to_num(7.0))
