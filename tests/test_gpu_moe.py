"""GPU parity of MoE routing (bit-exact integers) and the grouped expert FFN.

FFN bar: bf16 / fp16 within 2e-2 absolute of the host-engine oracle, or one
unit in the last place of the 16-bit result where that is larger (|y| >= 4 for
bf16: a GEMM whose fp32 summation order differs from ATen's flips the final
rounding of a few outputs, by exactly one ulp)."""
import ctypes as C

import pytest
import torch

import capi
import oracle as O
from conftest import assert_bit_exact
from ffn_bar import assert_ffn_close
from golden_util import DTYPE_TAGS, case

pytestmark = pytest.mark.gpu
NAMES = ("topi", "topw", "order", "inv", "counts", "offsets")


@pytest.mark.parametrize("tag", DTYPE_TAGS)
def test_route_golden(tag):
    c = case(f"moe_route_{tag}")
    got = capi.moe_route(c["logits"].cuda(), 2)
    for name, g in zip(NAMES, got):
        assert_bit_exact(g, c[name], f"moe_route {name}")


@pytest.mark.parametrize("shape", [(1, 8, 2), (100, 8, 2), (1000, 8, 2), (777, 16, 4), (300, 64, 8), (5000, 3, 3),
                                   (8192, 8, 2), (257, 1, 1), (4096, 8, 8), (1500, 32, 8), (999, 24, 3), (2100, 60, 7),
                                   (8192, 64, 8), (1000, 128, 8), (3000, 256, 8), (500, 200, 6), (70000, 128, 4)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_route_matches_oracle(shape, dtype):
    T, E, k = shape
    logits = torch.randn(T, E).to(dtype)
    if T > 10:
        logits[3] = logits[3, 0]                       # every expert tied
        logits[7, E // 2] = logits[7, 0]
    got = capi.moe_route(logits.cuda(), k)
    want = O.moe_route(logits, k)
    for name, g, w in zip(NAMES, got, want):
        assert_bit_exact(g, w, f"moe_route {name} T{T} E{E} k{k} {dtype}")


def test_route_quantised_logits_many_ties_and_skew():
    logits = torch.randint(-2, 3, (3000, 8)).float().bfloat16()     # 5 distinct values: ties everywhere
    logits[:, 5] += 5                                                 # one hot expert: skewed counts
    logits[:, 2] -= 9                                                 # one expert never chosen
    got = capi.moe_route(logits.cuda(), 2)
    want = O.moe_route(logits, 2)
    for name, g, w in zip(NAMES, got, want):
        assert_bit_exact(g, w, f"moe_route {name}")
    assert got[4][2].item() == 0 and got[4][5].item() == 3000


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T", [1, 7, 40, 64])
def test_ffn_few_rows_per_expert(T, dtype):
    """Decode-time batches run on the few-row kernels (a workgroup per 16 weight rows of an expert,
    the expert's rows 32 at a time): experts without a row, an expert with more than 32 rows (most
    tokens choose expert 3 first), a single token."""
    E, k, H, I = 8, 2, 256, 512
    torch.manual_seed(T)
    x = torch.randn(T, H).to(dtype)
    wg, wu, wd = (0.05 * torch.randn(E, I, H)).to(dtype), (0.05 * torch.randn(E, I, H)).to(dtype), (0.05 * torch.randn(E, H, I)).to(dtype)
    logits = torch.randn(T, E)
    logits[:, 3] += 6.0                    # everybody's first choice
    logits[:, 5:] -= 9.0                   # nobody's choice
    logits = logits.to(dtype)
    topi, topw, order, inv, counts, offsets = capi.moe_route(logits.cuda(), k)
    assert counts[3].item() == T and counts[5:].sum().item() == 0
    out = capi.moe_ffn(x.cuda(), wg.cuda(), wu.cuda(), wd.cuda(), topw, order, inv, offsets, k)
    want = O.moe_ffn(x, wg, wu, wd, topw.cpu(), order.cpu(), inv.cpu(), offsets.cpu(), k)
    assert_ffn_close(out, want, dtype)


def test_route_errors_and_empty():
    with pytest.raises(capi.ParasError, match="k out of range"):
        capi.moe_route(torch.randn(4, 8, device="cuda"), 9)
    topi, topw, order, inv, counts, offsets = capi.moe_route(torch.empty(0, 8, device="cuda"), 2)
    assert counts.tolist() == [0] * 8 and offsets.tolist() == [0] * 9


def test_ffn_golden():
    c = case("moe_ffn_bf16")
    d = {k: v.cuda() for k, v in c.items()}
    out = capi.moe_ffn(d["x"], d["wg"], d["wu"], d["wd"], d["topw"], d["order"], d["inv"], d["offsets"], 2)
    assert_ffn_close(out, c["out"], torch.bfloat16)


@pytest.mark.parametrize("shape", [(64, 4, 2, 128, 256), (300, 8, 2, 256, 512), (100, 8, 2, 128, 192), (257, 3, 1, 64, 64),
                                   (500, 8, 4, 320, 448), (333, 8, 3, 128, 128), (200, 16, 5, 64, 192), (150, 8, 7, 128, 64),
                                   (90, 12, 6, 192, 128)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_ffn_matches_oracle(shape, dtype):
    T, E, k, H, I = shape
    x, logits = torch.randn(T, H).to(dtype), torch.randn(T, E).to(dtype)
    logits[:, E - 1] -= 20                              # an expert that receives no token
    wg, wu = (0.05 * torch.randn(E, I, H)).to(dtype), (0.05 * torch.randn(E, I, H)).to(dtype)
    wd = (0.05 * torch.randn(E, H, I)).to(dtype)
    topi, topw, order, inv, counts, offsets = capi.moe_route(logits.cuda(), k)
    out = capi.moe_ffn(x.cuda(), wg.cuda(), wu.cuda(), wd.cuda(), topw, order, inv, offsets, k)
    r = O.moe_route(logits, k)
    want = O.moe_ffn(x, wg, wu, wd, r[1], r[2], r[3], r[5], k, gemm="aten")
    err = assert_ffn_close(out, want, dtype)
    assert err.mean().item() < 1e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(50, 3, 2, 72, 100), (33, 4, 1, 64, 40), (20, 2, 2, 7, 64)])
def test_ffn_sizes_the_tiles_do_not_take(shape, dtype):
    """Hidden or intermediate sizes that are not multiples of 64 run on the general kernels."""
    T, E, k, H, I = shape
    x, logits = torch.randn(T, H).to(dtype), torch.randn(T, E).to(dtype)
    wg, wu = (0.1 * torch.randn(E, I, H)).to(dtype), (0.1 * torch.randn(E, I, H)).to(dtype)
    wd = (0.1 * torch.randn(E, H, I)).to(dtype)
    topi, topw, order, inv, counts, offsets = capi.moe_route(logits.cuda(), k)
    out = capi.moe_ffn(x.cuda(), wg.cuda(), wu.cuda(), wd.cuda(), topw, order, inv, offsets, k)
    r = O.moe_route(logits, k)
    want = O.moe_ffn(x, wg, wu, wd, r[1], r[2], r[3], r[5], k, gemm="aten")
    assert_ffn_close(out, want, dtype)


def _at_offset(t, elems=1):
    """The same values in device memory that starts `elems` elements past an allocation's start."""
    flat = torch.empty(t.numel() + elems, dtype=t.dtype, device="cuda")
    view = flat[elems:].view(t.shape)
    view.copy_(t)
    return view


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_operands_that_are_not_16_byte_aligned(dtype):
    """A view at an odd storage offset: routing reads its 8-expert rows element by element and the FFN
    runs on the general kernels; same results as from aligned memory (routing exactly)."""
    T, E, k, H, I = 300, 8, 2, 128, 256
    x, logits = torch.randn(T, H).to(dtype), torch.randn(T, E).to(dtype)
    wg, wu = (0.05 * torch.randn(E, I, H)).to(dtype), (0.05 * torch.randn(E, I, H)).to(dtype)
    wd = (0.05 * torch.randn(E, H, I)).to(dtype)
    want_route = O.moe_route(logits, k)
    for elems in (1, 3):
        got = capi.moe_route(_at_offset(logits, elems), k)
        for g, w in zip(got, want_route):
            assert torch.equal(g.cpu(), w)
    topi, topw, order, inv, counts, offsets = capi.moe_route(logits.cuda(), k)
    want = O.moe_ffn(x, wg, wu, wd, want_route[1], want_route[2], want_route[3], want_route[5], k, gemm="aten")
    out = capi.moe_ffn(_at_offset(x), wg.cuda(), wu.cuda(), wd.cuda(), topw, order, inv, offsets, k)
    assert_ffn_close(out, want, dtype)
    out = capi.moe_ffn(x.cuda(), wg.cuda(), _at_offset(wu, 3), wd.cuda(), topw, order, inv, offsets, k)
    assert_ffn_close(out, want, dtype)


def test_config5_routing_exact_and_sampled_tokens():
    """BASELINE config 5 (T=8192 H=4096 E=8 top-2 I=14336 bf16) at full size:
    routing bit-exact on all tokens, the FFN on 48 sampled tokens against the
    oracle (a token's output depends only on its own row and routing)."""
    T, H, E, k, I = 8192, 4096, 8, 2, 14336
    dt = torch.bfloat16
    logits, x = torch.randn(T, E).to(dt), torch.randn(T, H).to(dt)
    wg, wu = (0.02 * torch.randn(E, I, H)).to(dt), (0.02 * torch.randn(E, I, H)).to(dt)
    wd = (0.02 * torch.randn(E, H, I)).to(dt)
    got = capi.moe_route(logits.cuda(), k)
    want = O.moe_route(logits, k)
    for name, g, w in zip(NAMES, got, want):
        assert_bit_exact(g, w, f"config 5 moe_route {name}")
    topi, topw, order, inv, counts, offsets = got
    out = capi.moe_ffn(x.cuda(), wg.cuda(), wu.cuda(), wd.cuda(), topw, order, inv, offsets, k)
    assert not bool(out.isnan().any())
    sel = torch.randperm(T)[:48]
    r = O.moe_route(logits[sel], k)
    ref = O.moe_ffn(x[sel], wg, wu, wd, r[1], r[2], r[3], r[5], k, gemm="aten")
    err = assert_ffn_close(out.cpu()[sel], ref, dt)
    assert err.mean().item() < 5e-4


def test_ffn_256_row_tiles_with_ragged_tiny_and_empty_experts():
    """Big enough for the 256-row tiles (8192 tokens, top-2, 5 experts of which one gets three
    tokens and one none): sampled tokens, all of the tiny expert's among them, against the oracle."""
    torch.manual_seed(5)
    T, H, E, k, I = 8192, 2048, 5, 2, 512
    dt = torch.bfloat16
    logits = torch.randn(T, E)
    logits[:, 3] -= 30.0                      # expert 3: only the three tokens below
    logits[:, 4] -= 60.0                      # expert 4: nobody
    tiny = torch.tensor([5, 4000, T - 1])
    logits[tiny, 3] += 60.0
    logits = logits.to(dt)
    x = torch.randn(T, H).to(dt)
    wg, wu = (0.03 * torch.randn(E, I, H)).to(dt), (0.03 * torch.randn(E, I, H)).to(dt)
    wd = (0.03 * torch.randn(E, H, I)).to(dt)
    topi, topw, order, inv, counts, offsets = capi.moe_route(logits.cuda(), k)
    assert counts.cpu().tolist()[3:] == [3, 0]
    out = capi.moe_ffn(x.cuda(), wg.cuda(), wu.cuda(), wd.cuda(), topw, order, inv, offsets, k)
    sel = torch.cat([tiny, torch.randperm(T)[:40]])
    r = O.moe_route(logits[sel], k)
    ref = O.moe_ffn(x[sel], wg, wu, wd, r[1], r[2], r[3], r[5], k, gemm="aten")
    assert_ffn_close(out.cpu()[sel], ref, dt)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_ffn_256_row_tiles_with_most_gates_outside_the_common_range(dtype):
    """Gates of standard deviation 14: four in ten lie below -8 or above 60, where SwiGLU is evaluated by
    its fp64 formula.  The 256-row kernel sets such values aside and works them off together; here they
    are most of the tile, more than can be set aside at once.  Sampled tokens against the oracle."""
    torch.manual_seed(23)
    T, H, E, k, I = 4096, 1024, 2, 2, 512          # (big enough for the 256-row tiles)
    logits = torch.randn(T, E).to(dtype)
    x = torch.randn(T, H).to(dtype)
    wg, wu = (0.45 * torch.randn(E, I, H)).to(dtype), (0.03 * torch.randn(E, I, H)).to(dtype)
    wd = (0.01 * torch.randn(E, H, I)).to(dtype)
    topi, topw, order, inv, counts, offsets = capi.moe_route(logits.cuda(), k)
    out = capi.moe_ffn(x.cuda(), wg.cuda(), wu.cuda(), wd.cuda(), topw, order, inv, offsets, k)
    sel = torch.randperm(T)[:64]
    r = O.moe_route(logits[sel], k)
    ref = O.moe_ffn(x[sel], wg, wu, wd, r[1], r[2], r[3], r[5], k, gemm="aten")
    assert float(ref.abs().max()) > 0.5
    assert_ffn_close(out.cpu()[sel], ref, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_ffn_256_row_tiles_with_nan_inf_and_zero_rows(dtype):
    """A NaN, an infinity and an all-zero row among the tokens of a layer big enough for the 256-row tiles:
    those tokens come out as the oracle has them (NaNs in the same places, exact zeros), and their
    neighbours in the same tiles are untouched."""
    torch.manual_seed(29)
    T, H, E, k, I = 4096, 1024, 2, 2, 512
    logits = torch.randn(T, E).to(dtype)
    x = torch.randn(T, H).to(dtype)
    x[5, 3] = float("nan")
    x[700, 10] = float("inf")
    x[1500] = 0
    wg, wu = (0.03 * torch.randn(E, I, H)).to(dtype), (0.03 * torch.randn(E, I, H)).to(dtype)
    wd = (0.03 * torch.randn(E, H, I)).to(dtype)
    topi, topw, order, inv, counts, offsets = capi.moe_route(logits.cuda(), k)
    out = capi.moe_ffn(x.cuda(), wg.cuda(), wu.cuda(), wd.cuda(), topw, order, inv, offsets, k).cpu()
    sel = torch.tensor([4, 5, 6, 699, 700, 701, 1499, 1500, 1501] + torch.randperm(T)[:23].tolist())
    r = O.moe_route(logits[sel], k)
    ref = O.moe_ffn(x[sel], wg, wu, wd, r[1], r[2], r[3], r[5], k, gemm="aten")
    got = out[sel]
    assert torch.equal(got.isnan(), ref.isnan())
    assert bool(ref[1].isnan().all()) and bool(ref[4].isnan().any())        # the NaN token, the infinite one
    assert torch.equal(got[7], torch.zeros(H, dtype=dtype)) and torch.equal(ref[7], torch.zeros(H, dtype=dtype))
    fin = ~ref.isnan().any(dim=1)
    assert int(fin.sum()) >= 30
    assert_ffn_close(got[fin], ref[fin], dtype)
    assert int(out.isnan().any(dim=1).sum()) == 2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_ffn_rows_in_the_last_tile_of_every_expert(dtype):
    """256-row tiles and experts whose last tiles hold 1, 40, 64, 65, 200 and 256 rows (a tile of at
    most 64 rows is shared out among the waves differently): every token with a row in some
    expert's last tile, and a few others, against the oracle."""
    torch.manual_seed(11)
    want_counts = [1025, 1064, 1088, 1089, 1224, 1280]
    E, k, H, I = len(want_counts), 2, 2048, 256
    T = sum(want_counts) // k
    rows = torch.repeat_interleave(torch.arange(E), torch.tensor(want_counts))   # token t: experts rows[t], rows[t + T]
    logits = 0.1 * torch.randn(T, E)
    logits[torch.arange(T), rows[:T]] += 5.0
    logits[torch.arange(T), rows[T:]] += 4.0
    perm = torch.randperm(T)
    logits = logits[perm].to(dtype)
    x = torch.randn(T, H).to(dtype)
    wg, wu = (0.03 * torch.randn(E, I, H)).to(dtype), (0.03 * torch.randn(E, I, H)).to(dtype)
    wd = (0.05 * torch.randn(E, H, I)).to(dtype)
    topi, topw, order, inv, counts, offsets = capi.moe_route(logits.cuda(), k)
    assert counts.cpu().tolist() == want_counts
    out = capi.moe_ffn(x.cuda(), wg.cuda(), wu.cuda(), wd.cuda(), topw, order, inv, offsets, k)
    off, ordr = offsets.cpu().tolist(), order.cpu()
    tails = [ordr[off[e] + (want_counts[e] - 1) // 256 * 256: off[e + 1]] // k for e in range(E)]
    sel = torch.unique(torch.cat(tails + [torch.randperm(T)[:32]]))
    r = O.moe_route(logits[sel], k)
    ref = O.moe_ffn(x[sel], wg, wu, wd, r[1], r[2], r[3], r[5], k, gemm="aten")
    assert_ffn_close(out.cpu()[sel], ref, dtype)


@pytest.mark.parametrize("shape", [(8192, 8, 2, torch.bfloat16), (5000, 64, 6, torch.float32), (700, 16, 4, torch.float16)])
def test_route_when_the_workgroups_do_not_wait_for_each_other(shape, monkeypatch):
    """With a wait of one poll most workgroups of the one-kernel routing stop waiting for the others
    and count every token's choices themselves (the path for a chip kept busy by unrelated work);
    the few that arrive last take the usual path.  Same outputs either way, bit for bit."""
    T, E, k, dtype = shape
    torch.manual_seed(T)
    logits = torch.randn(T, E).to(dtype)
    logits[5] = logits[5, 0]
    want = O.moe_route(logits, k)
    monkeypatch.setenv("PARAS_ROUTE_SPIN_LIMIT", "1")
    before, after = C.c_uint64(0), C.c_uint64(0)
    capi.check(capi.lib().paras_moe_route_give_ups(C.byref(before)))
    for _ in range(3):
        got = capi.moe_route(logits.cuda(), k)
        for name, g, w in zip(NAMES, got, want):
            assert_bit_exact(g, w, f"moe_route {name} without waiting")
    capi.check(capi.lib().paras_moe_route_give_ups(C.byref(after)))
    if T >= 5000:                                 # (a handful of workgroups may all have arrived by the first poll)
        assert after.value > before.value, "the give-up counter did not move"
    got = capi.moe_route_noalloc(logits.cuda(), k)
    for name, g, w in zip(NAMES, got, want):
        assert_bit_exact(g, w, f"moe_route_noalloc {name} without waiting")


def test_route_calls_of_changing_shapes_one_after_another():
    """The one-launch routing keeps its scratch inside the library and never clears it: what an
    earlier call of another shape left there must not count for a later one."""
    torch.manual_seed(77)
    for T, E, k, dtype in [(65536, 8, 2, torch.bfloat16), (300, 64, 8, torch.float32), (65536, 8, 2, torch.bfloat16),
                           (8192, 8, 2, torch.bfloat16), (65000, 64, 4, torch.float16), (8192, 8, 2, torch.bfloat16),
                           (1, 8, 2, torch.bfloat16), (257, 3, 1, torch.float32)]:
        logits = torch.randn(T, E).to(dtype)
        for _ in range(2):
            got = capi.moe_route(logits.cuda(), k)
            for name, g, w in zip(NAMES, got, O.moe_route(logits, k)):
                assert_bit_exact(g, w, f"moe_route {name} T{T} E{E} k{k}")


def test_route_on_a_callers_workspace_that_holds_stale_counts(monkeypatch):
    """PARAS_ROUTE_OWN_SCRATCH=0: the form used under graph capture.  The workspace is the caller's
    and may hold anything, here words that look like published counts: they are cleared first."""
    monkeypatch.setenv("PARAS_ROUTE_OWN_SCRATCH", "0")
    torch.manual_seed(78)
    for T, E, k, dtype in [(8192, 8, 2, torch.bfloat16), (3000, 64, 6, torch.float32)]:
        logits = torch.randn(T, E).to(dtype)
        n = capi.lib().paras_moe_route_workspace(T, E, k)
        ws = torch.empty((n + 7) // 8, dtype=torch.int64, device="cuda")
        for stale in ((1 << 16) | 77, -1):
            ws.fill_(stale)
            got = capi.moe_route(logits.cuda(), k, workspace=ws)
            for name, g, w in zip(NAMES, got, O.moe_route(logits, k)):
                assert_bit_exact(g, w, f"moe_route {name} on a workspace of stale words")


def test_route_calls_side_by_side_on_many_streams():
    """More streams than the library has scratch areas: calls that share one may see each other's
    epochs, wait their polls out and count for themselves.  Slow then, and still exact."""
    torch.manual_seed(79)
    k = 2
    streams = [torch.cuda.Stream() for _ in range(6)]
    inputs = [torch.randn(4096 + 512 * i, 8).bfloat16() for i in range(len(streams))]
    on_dev = [x.cuda() for x in inputs]
    torch.cuda.synchronize()
    results = []
    for _ in range(3):
        for s, x in zip(streams, on_dev):
            with torch.cuda.stream(s):
                results.append((x, capi.moe_route(x, k)))
    torch.cuda.synchronize()
    want = {id(x): O.moe_route(c, k) for x, c in zip(on_dev, inputs)}
    for x, got in results:
        for name, g, w in zip(NAMES, got, want[id(x)]):
            assert_bit_exact(g, w, f"moe_route {name} T{x.shape[0]} among other streams")


def test_route_recorded_into_a_graph_and_replayed():
    """A stream that is being captured gets the replayable form of the routing (a fill kernel clears
    the caller's workspace, no epoch from the host).  Replays with new logits, eager calls and
    synchronizations in between, each checked against the oracle."""
    torch.manual_seed(80)
    T, E, k = 8192, 8, 2
    static_logits = torch.randn(T, E).bfloat16().cuda()
    capi.moe_route(static_logits, k)                     # everything one-time is done before the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        recorded = capi.moe_route(static_logits, k)
    for trial in range(4):
        fresh = torch.randn(T, E).bfloat16()
        static_logits.copy_(fresh.cuda())
        eager = capi.moe_route(static_logits, k)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = O.moe_route(fresh, k)
        for name, g, e, w in zip(NAMES, recorded, eager, want):
            assert_bit_exact(g, w, f"replay {trial}: moe_route {name}")
            assert_bit_exact(e, w, f"eager call {trial}: moe_route {name}")
