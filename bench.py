#!/usr/bin/env python3
"""Benchmark of the fused transformer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]

Prints ONE JSON line.  The headline value is BASELINE.json's first metric:
bf16 causal flash-attention forward at B=4, H=32, S=4096, D=128 (configs[2]) in
TFLOP/s, counted with the causal-halved figure 4*B*H*S^2*D/2.  The same line
carries, under "workloads", the other configurations the metric names
(RMSNorm and SwiGLU of configs[1] in GB/s, the GQA decode of configs[3], the
MoE layer of configs[4]), the dense projection GEMM and the backward / RoPE
helper ops that sit either side of the path, each with its own roofline object.

A step is one pass of the workload's kernels over one batch of synthetic
inputs (seeded N(0,1) / N(1,0.02) / N(0,0.02) as BASELINE.json states) that
are resident in HBM before the timed region.  Kernels are called through the C
ABI of libparas_hip.so on torch's current stream; per-launch durations come
from HIP events recorded on that same stream.  The HBM-bound kernels rotate
over enough buffers that no input is served from the 256 MB last-level cache.

cpu_baseline times the reference's own CPU flavor (oracle/_ref, "reference")
-- or, if that library is absent, the oracle's C restatement ("port") -- on a
bounded sample of the headline workload in a child process on this box's host
cores.  It is a reported baseline, not a target.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for p in (ROOT / "tests", ROOT / "oracle"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))

HBM_PEAK_GBS = 8000.0         # MI355X published HBM3E bandwidth
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 MFMA rate
METRIC = "SDPA TFLOP/s (% MFMA peak); RMSNorm/SwiGLU GB/s (% HBM peak) at 1 GPU"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def load_traffic() -> dict:
    """HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE, then
    WRITE_SIZE, each scaled by what the same counter reads for the `copy`
    workload of known size), recorded next to the profile summaries as lines
    "<kernel> <fetch bytes> <write bytes>"."""
    path = ROOT / "profiles" / "hbm_traffic.txt"
    out = {}
    if path.exists():
        for ln in path.read_text().splitlines():
            f = ln.split()
            if len(f) == 3 and not ln.startswith("#"):
                out[f[0]] = int(float(f[1]) + float(f[2]))
    return out


SETTLE_MS = 40.0        # untimed settling of the short memory-bound launches (see Timer.run)


class Timer:
    """HIP events on the launch stream: average launch duration in ms."""

    def __init__(self, torch):
        self.torch = torch

    def run(self, fn, steps, warmup, settle_ms=0.0):
        """`warmup` untimed calls, then exactly `steps` timed ones.  `settle_ms` > 0 keeps
        making untimed calls until that much wall time has passed: a launch of 50 us
        measured after 25 warm-up calls is still on the memory clocks' ramp (the first
        ~25 ms of work after an idle gap run about 10 % slower)."""
        torch = self.torch
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        t_settle = time.perf_counter()
        while settle_ms > 0 and (time.perf_counter() - t_settle) * 1e3 < settle_ms:
            for i in range(16):
                fn(i)
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for i in range(steps):
            fn(warmup + i)
        e1.record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
        return e0.elapsed_time(e1) / steps, wall_ms


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=200)     # steady clocks: the first ~100 ms of launches after an idle gap run 1-2 % slower
    ap.add_argument("--workload", default="all",
                    choices=["all", "sdpa_prefill", "rmsnorm_swiglu", "sdpa_decode", "moe", "linear", "backward_ops", "copy"],
                    help="'copy' is the counter calibration: a plain 1 GiB device copy, not part of 'all'")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build targets one GPU; --gpus must be 1 (nothing here shards across GPUs)", file=sys.stderr)
        return 2

    import torch
    import capi

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    L = capi.lib()                       # raises if libparas_hip.so is missing: no fallback
    assert L.paras_device_count() >= 1
    torch.manual_seed(0)
    dev = "cuda:0"
    bf = torch.bfloat16
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    timer = Timer(torch)
    traffic = load_traffic()
    steps, warmup = args.steps, args.warmup
    want = lambda name: args.workload in ("all", name)
    results = {}

    def must(rc):
        if rc != 0:
            raise RuntimeError(L.paras_last_error().decode())

    def roofline(bound, achieved, key):
        peak = HBM_PEAK_GBS if bound == "hbm" else MFMA_BF16_PEAK_TFLOPS
        return {"bound": bound, "achieved": round(achieved, 2), "peak": peak,
                "unit": "GB/s" if bound == "hbm" else "TFLOP/s", "frac": round(achieved / peak, 4),
                "traffic": traffic.get(key)}

    # ------------------------------------------------------------------ configs[2]
    if want("sdpa_prefill"):
        B, H, S, D = 4, 32, 4096, 128
        q, k, v = (torch.randn(B, H, S, D, device=dev).to(bf) for _ in range(3))
        out = torch.empty_like(q)
        a = capi.sdpa_args(q, k, v, out, is_causal=True)
        assert L.paras_sdpa_kernel_name(C.byref(a)) == b"flash_mfma"
        ms, wall = timer.run(lambda i: must(L.paras_sdpa_fwd(C.byref(a), None, st)), steps, warmup)
        flops = 4 * B * H * S * S * D / 2          # causal-halved
        tf = flops / ms / 1e9
        results["sdpa_prefill"] = {
            "workload": "bf16 causal flash-attention fwd B=4 H=32 S=4096 D=128 (configs[2])",
            "value": round(tf, 2), "unit": "TFLOP/s", "ms_per_step": round(ms, 4), "wall_ms_per_step": round(wall, 4),
            "kernel": "flash_fwd_kernel<bf16,128,causal>", "algorithmic_flops_per_launch": flops,
            "roofline": roofline("mfma", tf, "flash_fwd_kernel"),
        }
        log(f"sdpa_prefill: {ms * 1e3:.1f} us  {tf:.1f} TFLOP/s  ({tf / MFMA_BF16_PEAK_TFLOPS:.1%} of dense bf16 peak)")
        del q, k, v, out

    # ------------------------------------------------------------------ configs[1]
    if want("rmsnorm_swiglu"):
        rows, Hd, I = 16384, 4096, 14336
        nrot = 4                                  # 4 x 268 MB of RMSNorm traffic between reuses of a buffer
        xs = [torch.randn(rows, Hd, device=dev).to(bf) for _ in range(nrot)]
        outs = [torch.empty_like(x) for x in xs]
        w = (1 + 0.02 * torch.randn(Hd, device=dev)).to(bf)
        rstd = torch.empty(rows, dtype=torch.float32, device=dev)

        def rms(i):
            j = i % nrot
            must(L.paras_rms_norm_fwd(xs[j].data_ptr(), w.data_ptr(), outs[j].data_ptr(), rstd.data_ptr(), rows, Hd,
                                      1e-6, capi.BF16, st))
        ms_r, _ = timer.run(rms, steps, warmup, SETTLE_MS)
        bytes_r = 2 * rows * Hd * 2 + Hd * 2 + rows * 4
        gbs_r = bytes_r / ms_r / 1e6
        del xs, outs
        gate = torch.randn(rows, I, device=dev).to(bf)
        up = torch.randn(rows, I, device=dev).to(bf)
        so = torch.empty_like(gate)
        n = rows * I
        ms_s, _ = timer.run(lambda i: must(L.paras_swiglu_fwd(gate.data_ptr(), up.data_ptr(), so.data_ptr(), n, capi.BF16, st)),
                            steps, warmup, SETTLE_MS)
        bytes_s = 3 * n * 2
        gbs_s = bytes_s / ms_s / 1e6
        results["rmsnorm_swiglu"] = {
            "workload": "bf16 fused RMSNorm 16384x4096 (eps 1e-6) then SwiGLU 16384x14336 (configs[1])",
            "value": round((bytes_r + bytes_s) / (ms_r + ms_s) / 1e6, 1), "unit": "GB/s",
            "ms_per_step": round(ms_r + ms_s, 4),
            "rms_norm": {"ms": round(ms_r, 4), "algorithmic_bytes_per_launch": bytes_r, "kernel": "rms_norm_fwd_vec<bf16,2>",
                         "roofline": roofline("hbm", gbs_r, "rms_norm_fwd_vec")},
            "swiglu": {"ms": round(ms_s, 4), "algorithmic_bytes_per_launch": bytes_s, "kernel": "swiglu_fwd_vec<bf16>",
                       "roofline": roofline("hbm", gbs_s, "swiglu_fwd_vec")},
        }
        log(f"rms_norm: {ms_r * 1e3:.1f} us  {gbs_r:.0f} GB/s ({gbs_r / HBM_PEAK_GBS:.1%})   "
            f"swiglu: {ms_s * 1e3:.1f} us  {gbs_s:.0f} GB/s ({gbs_s / HBM_PEAK_GBS:.1%})")
        del gate, up, so

    # ------------------------------------------------------------------ configs[3]
    if want("sdpa_decode"):
        B, Hq, Hkv, Lk, D = 64, 32, 8, 8192, 128
        q = torch.randn(B, Hq, 1, D, device=dev).to(bf)
        k, v = torch.randn(B, Hkv, Lk, D, device=dev).to(bf), torch.randn(B, Hkv, Lk, D, device=dev).to(bf)
        out = torch.empty_like(q)
        a = capi.sdpa_args(q, k, v, out)
        assert L.paras_sdpa_kernel_name(C.byref(a)) == b"decode_split"
        ws = torch.empty(max(1, L.paras_sdpa_workspace(C.byref(a))), dtype=torch.uint8, device=dev)
        ms, _ = timer.run(lambda i: must(L.paras_sdpa_fwd(C.byref(a), C.c_void_p(ws.data_ptr()), st)), steps, warmup, SETTLE_MS)
        nbytes = 2 * B * Hkv * Lk * D * 2 + 2 * B * Hq * D * 2
        gbs = nbytes / ms / 1e6
        results["sdpa_decode"] = {
            "workload": "bf16 GQA decode SDPA B=64 Hq=32 Hkv=8 Lq=1 Lk=8192 D=128 (configs[3])",
            "value": round(gbs, 1), "unit": "GB/s", "ms_per_step": round(ms, 4),
            "tokens_per_s": round(B / ms * 1e3, 1), "kernel": "decode_split_kernel<bf16> + decode_combine_kernel",
            "algorithmic_bytes_per_launch": nbytes, "roofline": roofline("hbm", gbs, "decode_split_kernel"),
        }
        log(f"sdpa_decode: {ms * 1e3:.1f} us  {gbs:.0f} GB/s ({gbs / HBM_PEAK_GBS:.1%})")
        del q, k, v, out, ws

    # ------------------------------------------------------------------ configs[4]
    if want("moe"):
        T, Hd, E, kk, I = 8192, 4096, 8, 2, 14336
        x = torch.randn(T, Hd, device=dev).to(bf)
        logits = torch.randn(T, E, device=dev).to(bf)
        wg = (0.02 * torch.randn(E, I, Hd, device=dev)).to(bf)
        wu = (0.02 * torch.randn(E, I, Hd, device=dev)).to(bf)
        wd = (0.02 * torch.randn(E, Hd, I, device=dev)).to(bf)
        topi = torch.empty(T, kk, dtype=torch.int64, device=dev)
        topw = torch.empty(T, kk, dtype=torch.float32, device=dev)
        order = torch.empty(T * kk, dtype=torch.int64, device=dev)
        inv = torch.empty_like(order)
        counts = torch.empty(E, dtype=torch.int64, device=dev)
        offsets = torch.empty(E + 1, dtype=torch.int64, device=dev)
        rws = torch.empty(max(1, L.paras_moe_route_workspace(T, E, kk)), dtype=torch.uint8, device=dev)
        fws = torch.empty(L.paras_moe_ffn_workspace(T, kk, Hd, I, capi.BF16), dtype=torch.uint8, device=dev)
        out = torch.empty(T, Hd, dtype=bf, device=dev)

        def route(i):
            must(L.paras_moe_route(logits.data_ptr(), T, E, kk, capi.BF16, topi.data_ptr(), topw.data_ptr(), order.data_ptr(),
                                   inv.data_ptr(), counts.data_ptr(), offsets.data_ptr(), rws.data_ptr(), st))

        def ffn(i):
            must(L.paras_moe_ffn(x.data_ptr(), wg.data_ptr(), wu.data_ptr(), wd.data_ptr(), topw.data_ptr(), order.data_ptr(),
                                 inv.data_ptr(), offsets.data_ptr(), out.data_ptr(), fws.data_ptr(), T, E, kk, Hd, I, capi.BF16, st))
        msteps, mwarm = max(3, steps // 5), max(1, warmup // 5)
        ms_route, _ = timer.run(route, msteps, mwarm)
        ms_ffn, _ = timer.run(ffn, msteps, mwarm)
        ms_all, _ = timer.run(lambda i: (route(i), ffn(i)), msteps, mwarm)
        flops = T * kk * 3 * 2 * Hd * I
        tf = flops / ms_ffn / 1e9
        results["moe"] = {
            "workload": "bf16 MoE layer T=8192 H=4096 E=8 top-2 I=14336: routing + grouped expert FFN (configs[4])",
            "value": round(T / ms_all * 1e3, 1), "unit": "tokens/s", "ms_per_step": round(ms_all, 4),
            "route_ms": round(ms_route, 4), "ffn_ms": round(ms_ffn, 4), "ffn_tflops": round(tf, 2),
            "kernel": "grouped_gemm_kernel<bf16> (gate-up+SwiGLU, down) + moe_combine_kernel",
            "algorithmic_flops_per_launch": flops, "roofline": roofline("mfma", tf, "grouped_gemm_kernel"),
        }
        log(f"moe: route {ms_route * 1e3:.1f} us, ffn {ms_ffn * 1e3:.1f} us = {tf:.1f} TFLOP/s ({tf / MFMA_BF16_PEAK_TFLOPS:.1%}), "
            f"layer {ms_all * 1e3:.1f} us = {T / ms_all * 1e3:.0f} tokens/s")
        del x, wg, wu, wd, fws, out

    # ------------------------------------------------------------------ dense projection (the callers either side of the path)
    if want("linear"):
        M, N, K = 16384, 4096, 4096               # 4 x 4096 tokens through a hidden x hidden nn.Linear
        xa = torch.randn(M, K, device=dev).to(bf)
        wb = (0.02 * torch.randn(N, K, device=dev)).to(bf)
        yc = torch.empty(M, N, dtype=bf, device=dev)
        ms, _ = timer.run(lambda i: must(L.paras_gemm_nt(xa.data_ptr(), wb.data_ptr(), None, yc.data_ptr(), M, N, K, K, K, N, 0,
                                                         1, 0, 0, 0, 0, 1.0, 0.0, capi.BF16, st)), steps, warmup)
        flops = 2 * M * N * K
        tf = flops / ms / 1e9
        results["linear"] = {
            "workload": "bf16 dense NT GEMM x W^T: M=16384 N=4096 K=4096 (nn.Linear of configs[2]'s tokens)",
            "value": round(tf, 2), "unit": "TFLOP/s", "ms_per_step": round(ms, 4), "kernel": "dense_gemm_nt_kernel<bf16>",
            "algorithmic_flops_per_launch": flops, "roofline": roofline("mfma", tf, "dense_gemm_nt_kernel"),
        }
        log(f"linear: {ms * 1e3:.1f} us  {tf:.1f} TFLOP/s ({tf / MFMA_BF16_PEAK_TFLOPS:.1%})")
        del xa, wb, yc

    # ------------------------------------------------------------------ the ops either side of the path
    if want("backward_ops"):
        rows, Hd, I = 16384, 4096, 14336
        nrot = 3                                  # every buffer is out of the 256 MB last-level cache when it comes round again
        xb = [torch.randn(rows, Hd, device=dev).to(bf) for _ in range(nrot)]
        gob = [torch.randn(rows, Hd, device=dev).to(bf) for _ in range(nrot)]
        w = (1 + 0.02 * torch.randn(Hd, device=dev)).to(bf)
        y, gw = torch.empty_like(xb[0]), torch.empty_like(w)
        gxb = [torch.empty_like(xb[0]) for _ in range(nrot)]
        rstd = torch.empty(rows, dtype=torch.float32, device=dev)
        # rows of every buffer are drawn from the same distribution: one rstd serves the timing of all three
        must(L.paras_rms_norm_fwd(xb[0].data_ptr(), w.data_ptr(), y.data_ptr(), rstd.data_ptr(), rows, Hd, 1e-6, capi.BF16, st))
        ws = torch.empty(L.paras_rms_norm_bwd_workspace(rows, Hd), dtype=torch.uint8, device=dev)
        ms_b, _ = timer.run(lambda i: must(L.paras_rms_norm_bwd(gob[i % nrot].data_ptr(), xb[i % nrot].data_ptr(), w.data_ptr(),
                                                                 rstd.data_ptr(), gxb[i % nrot].data_ptr(), gw.data_ptr(),
                                                                 ws.data_ptr(), rows, Hd, capi.BF16, st)),
                            steps, warmup, SETTLE_MS)
        bytes_b = 3 * rows * Hd * 2 + rows * 4 + 2 * Hd * 2
        del y, gxb, xb, gob, ws
        gate = torch.randn(rows, I, device=dev).to(bf)
        up = torch.randn(rows, I, device=dev).to(bf)
        g2 = torch.randn(rows, I, device=dev).to(bf)
        dg, du = torch.empty_like(gate), torch.empty_like(gate)
        n = rows * I
        ms_s, _ = timer.run(lambda i: must(L.paras_swiglu_bwd(g2.data_ptr(), gate.data_ptr(), up.data_ptr(), dg.data_ptr(),
                                                               du.data_ptr(), n, capi.BF16, st)), steps, warmup, SETTLE_MS)
        bytes_s = 5 * n * 2
        del gate, up, g2, dg, du
        qhs = [torch.randn(4 * 32 * 4096, 128, device=dev).to(bf) for _ in range(4)]
        qos = [torch.empty_like(q_) for q_ in qhs]
        qh = qhs[0]
        ms_r, _ = timer.run(lambda i: must(L.paras_rotate_half(qhs[i % 4].data_ptr(), qos[i % 4].data_ptr(), qh.shape[0], 128, 0,
                                                               capi.BF16, st)), steps, warmup, SETTLE_MS)
        bytes_r = 2 * qh.numel() * 2
        gb = lambda b, ms: b / ms / 1e6
        results["backward_ops"] = {
            "workload": "bf16 RMSNorm backward 16384x4096, SwiGLU backward 16384x14336, rotate_half 4x32x4096x128",
            "value": round((bytes_b + bytes_s + bytes_r) / (ms_b + ms_s + ms_r) / 1e6, 1), "unit": "GB/s",
            "ms_per_step": round(ms_b + ms_s + ms_r, 4),
            "rms_norm_bwd": {"ms": round(ms_b, 4), "algorithmic_bytes_per_launch": bytes_b,
                             "kernel": "rms_norm_bwd_fused<bf16,1,512> + rms_norm_bwd_dw_final_wide",
                             "roofline": roofline("hbm", gb(bytes_b, ms_b), "rms_norm_bwd_fused")},
            "swiglu_bwd": {"ms": round(ms_s, 4), "algorithmic_bytes_per_launch": bytes_s, "kernel": "swiglu_bwd_vec<bf16>",
                           "roofline": roofline("hbm", gb(bytes_s, ms_s), "swiglu_bwd_vec")},
            "rotate_half": {"ms": round(ms_r, 4), "algorithmic_bytes_per_launch": bytes_r, "kernel": "rotate_half_vec16",
                            "roofline": roofline("hbm", gb(bytes_r, ms_r), "rotate_half_vec16")},
        }
        log(f"backward_ops: rms_norm_bwd {ms_b * 1e3:.1f} us {gb(bytes_b, ms_b):.0f} GB/s ({gb(bytes_b, ms_b) / HBM_PEAK_GBS:.1%})   "
            f"swiglu_bwd {ms_s * 1e3:.1f} us {gb(bytes_s, ms_s):.0f} GB/s ({gb(bytes_s, ms_s) / HBM_PEAK_GBS:.1%})   "
            f"rotate_half {ms_r * 1e3:.1f} us {gb(bytes_r, ms_r):.0f} GB/s ({gb(bytes_r, ms_r) / HBM_PEAK_GBS:.1%})")
        del qh, qhs, qos

    # ------------------------------------------------------------------ counter calibration
    if args.workload == "copy":
        n = 1 << 29                                # 2^29 bf16 elements: 1 GiB read + 1 GiB written
        src = torch.randn(n // 4096, 4096, device=dev).to(bf)
        dst = torch.empty_like(src)
        shape, stride = (C.c_int64 * 1)(n), (C.c_int64 * 1)(1)
        ms, _ = timer.run(lambda i: must(L.paras_copy_strided(src.data_ptr(), dst.data_ptr(), 1, shape, stride, stride, 2,
                                                              capi.BF16, capi.BF16, st)), steps, warmup)
        gbs = 4 * n / ms / 1e6
        results["copy"] = {"workload": "plain device copy of 2^29 bf16 elements (counter calibration)", "value": round(gbs, 1),
                           "unit": "GB/s", "ms_per_step": round(ms, 4), "kernel": "copy kernel", "algorithmic_bytes_per_launch": 4 * n,
                           "roofline": roofline("hbm", gbs, "copy")}
        log(f"copy: {ms * 1e3:.1f} us  {gbs:.0f} GB/s ({gbs / HBM_PEAK_GBS:.1%})")

    # ------------------------------------------------------------------ cpu baseline
    head_name = "sdpa_prefill" if "sdpa_prefill" in results else next(iter(results))
    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(head_name)

    head = results[head_name]
    line = {
        "metric": METRIC,
        "value": head["value"],
        "unit": head["unit"],
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": head["workload"], "device": torch.cuda.get_device_name(0),
                   "timing": "HIP events on the launch stream, inputs resident in HBM"},
        "roofline": head.get("roofline") or next(v["roofline"] for v in head.values() if isinstance(v, dict) and "roofline" in v),
        "cpu_baseline": cpu,
        "workloads": results,
    }
    print(json.dumps(line))
    return 0


def cpu_baseline(name: str):
    """Times a bounded sample of the workload on the host cores: the reference's
    own CPU flavor when oracle/_ref is present, else the oracle's restatement."""
    import ref_engine as R
    samples = {
        "sdpa_prefill": ({"B": 4, "H": 32, "S": 4096, "D": 128}, lambda s: 4 * s["B"] * s["H"] * s["S"] ** 2 * s["D"] / 2 / 1e12, "TFLOP/s",
                         "the whole workload once: B=4, H=32, S=4096, D=128"),
        "rmsnorm_swiglu": ({"rows": 2048, "H": 4096, "I": 14336}, lambda s: (2 * s["rows"] * s["H"] * 2 + 3 * s["rows"] * s["I"] * 2) / 1e9, "GB/s",
                           "2048 of the 16384 rows (1/8 of the workload)"),
        "sdpa_decode": ({"B": 2, "Hq": 32, "Hkv": 8, "Lk": 8192, "D": 128}, lambda s: 2 * s["B"] * s["Hkv"] * s["Lk"] * s["D"] * 2 / 1e9, "GB/s",
                        "B=2 of 64 sequences (1/32 of the workload)"),
        "moe": ({"T": 128, "H": 4096, "E": 8, "k": 2, "I": 14336}, lambda s: s["T"] / 1.0, "tokens/s",
                "128 of the 8192 tokens, all 8 experts' weights"),
    }
    sample, work, unit, text = samples[name]
    try:
        if R.available():
            res = R.run("time_workload", name, sample)
            threads = R.run("host_threads")
            kind = "reference"
        else:
            res, threads, kind = port_baseline(name, sample)
        val = work(sample) / res["seconds"]
        log(f"cpu_baseline[{kind}] {name}: sample took {res['seconds']:.2f} s on {threads} threads -> {val:.4g} {unit}")
        return {"value": float(f"{val:.4g}"), "unit": unit, "cores": threads, "kind": kind,
                "sample": f"{text}; {res['seconds']:.2f} s of CPU work", "detail": res}
    except Exception as e:  # the baseline is informative; its failure must not hide the GPU result
        log(f"cpu_baseline failed: {e}")
        return {"value": None, "unit": unit, "cores": os.cpu_count(), "kind": "unavailable", "sample": str(e)[:200]}


def port_baseline(name, sample):
    import torch
    import oracle as O
    torch.manual_seed(0)
    bf = torch.bfloat16
    if name != "sdpa_prefill":
        raise RuntimeError("oracle/_ref missing and the port baseline covers sdpa_prefill only")
    B, H, S, D = sample["B"], sample["H"], sample["S"], sample["D"]
    q, k, v = (torch.randn(B, H, S, D).to(bf) for _ in range(3))
    t0 = time.perf_counter()
    O.sdpa_math(q, k, v, is_causal=True, gemm="aten")
    return {"seconds": time.perf_counter() - t0}, O.get_threads(), "port"


if __name__ == "__main__":
    sys.exit(main())
