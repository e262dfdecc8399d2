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
inputs that are resident in HBM before the timed region.  Inputs are drawn the
way the reference's tests draw theirs: torch.manual_seed(0) at the start of
each workload, torch-CPU randn (N(0,1) / N(1,0.02) / N(0,0.02) as BASELINE.json
states), then moved to the device.  Kernels are called through the C ABI of
libparas_hip.so on torch's current stream; per-launch durations come from HIP
events recorded on that same stream.  Every workload first makes untimed
launches for a fixed wall time (SETTLE_MS / SETTLE_MFMA_MS, whatever --warmup
says) so that the clocks have settled when the timed launches start.  The
HBM-bound kernels rotate over enough buffers that no input is served from the
256 MB last-level cache.

The cpu_baseline leg does two things per workload, both outside the timed
region: it times the reference's own CPU flavor (oracle/_ref, "reference") --
or, if that library is absent, the oracle's C restatement ("port") -- on a
bounded sample of the workload in a child process on this box's host cores, and
it compares a slice of the output the timed launches produced with the oracle
("parity").  The baseline is a reported figure, not a target.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import math
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for p in (ROOT / "framework-torch-paras_amd", ROOT / "oracle"):
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
        measured_on = None
        for ln in path.read_text().splitlines():
            f = ln.split()
            if ln.startswith("# kernel sources "):
                measured_on = f[3]
            elif len(f) == 3 and not ln.startswith("#"):
                out[f[0]] = int(float(f[1]) + float(f[2]))
        now = kernel_sources_digest()
        if measured_on != now:
            log(f"bench.py: profiles/hbm_traffic.txt was measured on kernel sources {measured_on}, the tree holds {now}: "
                "the `traffic` figures may be stale (measure again with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)")
            out["_stale"] = True
    return out


def kernel_sources_digest() -> str:
    """Digest of the kernel sources the library is built from; the traffic file records the one it was measured on."""
    import hashlib
    h = hashlib.sha256()
    for f in sorted((ROOT / "framework-torch-paras_amd" / "csrc").rglob("*")):
        if f.suffix in (".hip", ".h", ".cpp"):
            h.update(f.name.encode())
            h.update(f.read_bytes())
    return h.hexdigest()[:16]


SETTLE_MS = 40.0        # untimed settling of the short memory-bound launches (see Timer.run)
SETTLE_MFMA_MS = 300.0  # the matrix kernels: the first launches after an idle gap run up to 30 % slower, the first ~100 ms 1-2 %


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
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--workload", default="all",
                    choices=["all", "sdpa_prefill", "sdpa_weights", "rmsnorm_swiglu", "sdpa_decode", "moe", "linear", "backward_ops", "copy"],
                    help="'copy' is the counter calibration: a plain 1 GiB device copy, not part of 'all'")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg (baseline timing and parity check)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build targets one GPU; --gpus must be 1 (nothing here shards across GPUs)", file=sys.stderr)
        return 2

    import torch
    import paras_capi as capi

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    L = capi.lib()                       # raises if libparas_hip.so is missing: no fallback
    assert L.paras_device_count() >= 1
    dev = "cuda:0"
    bf = torch.bfloat16
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    timer = Timer(torch)
    traffic = load_traffic()
    steps, warmup = args.steps, args.warmup
    want = lambda name: args.workload in ("all", name)
    results = {}
    checks = {}      # workload -> closure run by the cpu leg: compares a slice of the timed output with the oracle

    def must(rc):
        if rc != 0:
            raise RuntimeError(L.paras_last_error().decode())

    def roofline(bound, achieved, key):
        peak = HBM_PEAK_GBS if bound == "hbm" else MFMA_BF16_PEAK_TFLOPS
        return {"bound": bound, "achieved": round(achieved, 2), "peak": peak,
                "unit": "GB/s" if bound == "hbm" else "TFLOP/s", "frac": round(achieved / peak, 4),
                "traffic": traffic.get(key)}

    def draw(*shape, mean=0.0, std=1.0, dtype=bf):
        """torch-CPU randn from the generator seeded at the start of the workload, narrowed on the host."""
        t = torch.randn(*shape)
        if std != 1.0:
            t *= std
        if mean != 0.0:
            t += mean
        return t.to(dtype)

    # ------------------------------------------------------------------ configs[2]
    if want("sdpa_prefill"):
        torch.manual_seed(0)
        B, H, S, D = 4, 32, 4096, 128
        qc, kc, vc = draw(B, H, S, D), draw(B, H, S, D), draw(B, H, S, D)
        q, k, v = qc.to(dev), kc.to(dev), vc.to(dev)
        out = torch.empty_like(q)
        a = capi.sdpa_args(q, k, v, out, is_causal=True)
        kname = L.paras_sdpa_kernel_name(C.byref(a)).decode()
        assert kname.startswith("flash_mfma")
        wide = kname == "flash_mfma_wide"      # 64 queries per wavefront, one workgroup per CU walking a list of items
        ms, wall = timer.run(lambda i: must(L.paras_sdpa_fwd(C.byref(a), None, st)), steps, warmup, SETTLE_MFMA_MS)
        flops = 4 * B * H * S * S * D / 2          # causal-halved
        tf = flops / ms / 1e9
        results["sdpa_prefill"] = {
            "workload": "bf16 causal flash-attention fwd B=4 H=32 S=4096 D=128 (configs[2])",
            "value": round(tf, 2), "unit": "TFLOP/s", "ms_per_step": round(ms, 4), "wall_ms_per_step": round(wall, 4),
            "kernel": "flash_wide_kernel<bf16,causal>" if wide else "flash_fwd_kernel<bf16,128,causal>",
            "algorithmic_flops_per_launch": flops,
            "roofline": roofline("mfma", tf, "flash_wide_kernel" if wide else "flash_fwd_kernel"),
        }
        log(f"sdpa_prefill: {ms * 1e3:.1f} us  {tf:.1f} TFLOP/s  ({tf / MFMA_BF16_PEAK_TFLOPS:.1%} of dense bf16 peak)")
        # What this box sustains on a register-only loop of the same MFMA (random operands): the published
        # peak assumes 2.4 GHz, under MFMA load the part is power limited.  Reported, not used in `frac`.
        sustained = {}
        for label, wps, valu in (("one_wave_per_simd", 1, 0), ("two_waves_per_simd", 2, 0), ("two_waves_per_simd_2_fp32_per_mfma", 2, 2)):
            rate = C.c_double(0.0)
            must(L.paras_mfma_rate_probe(wps, valu, C.byref(rate)))
            sustained[label] = round(rate.value, 1)
        results["sdpa_prefill"]["mfma_loop_tflops_on_this_box"] = sustained
        log(f"  register-only MFMA loop on this box: {sustained} TFLOP/s; the flash kernel runs one wavefront per SIMD")
        got_head = [(b_, h_, out[b_, h_, :256].cpu()) for b_, h_ in ((0, 0), (3, 31))]
        got_tail = out[1, 7, S - 64:].cpu()

        def check_prefill(O, qc=qc, kc=kc, vc=vc, got_head=got_head, got_tail=got_tail, S=S):
            worst = 0.0
            for b_, h_, got in got_head:     # a causal query sees its prefix only: the first 256 queries of a head stand alone
                ref, _ = O.sdpa_math(qc[b_:b_ + 1, h_:h_ + 1, :256], kc[b_:b_ + 1, h_:h_ + 1, :256], vc[b_:b_ + 1, h_:h_ + 1, :256],
                                     is_causal=True, gemm="aten")
                worst = max(worst, (got.float() - ref[0, 0].float()).abs().max().item())
            rows = torch.arange(S - 64, S)   # the last 64 queries of another head against all keys (the causal rule as a bool mask)
            allow = torch.arange(S)[None, :] <= rows[:, None]
            ref, _ = O.sdpa_math(qc[1:2, 7:8, S - 64:], kc[1:2, 7:8], vc[1:2, 7:8], attn_mask=allow, gemm="aten")
            worst = max(worst, (got_tail.float() - ref[0, 0].float()).abs().max().item())
            return {"max_abs_err": worst, "tolerance": 2e-2, "ok": worst <= 2e-2,
                    "slice": "queries 0..255 of heads (0,0) and (3,31), queries 4032..4095 of head (1,7)"}
        checks["sdpa_prefill"] = check_prefill
        del q, k, v, out

    # ------------------------------------------------------------------ the math op with its weights returned
    if want("sdpa_weights"):
        torch.manual_seed(0)
        B, H, S, D = 2, 16, 2048, 128
        qc, kc, vc = draw(B, H, S, D), draw(B, H, S, D), draw(B, H, S, D)
        q, k, v = qc.to(dev), kc.to(dev), vc.to(dev)
        out = torch.empty_like(q)
        attn = torch.empty(B, H, S, S, dtype=bf, device=dev)
        scale = float(torch.tensor(D ** -0.5).to(bf))          # narrowed to the tensors' dtype, as the op layer passes it
        a = capi.sdpa_args(q, k, v, out, attn=attn, is_causal=True, scale=scale)
        assert L.paras_sdpa_kernel_name(C.byref(a)) == b"math_mfma"
        ms, wall = timer.run(lambda i: must(L.paras_sdpa_fwd(C.byref(a), None, st)), steps, warmup, SETTLE_MFMA_MS)
        nbytes = attn.numel() * 2 + 4 * q.numel() * 2          # the weights written, q / k / v read, out written
        gbs = nbytes / ms / 1e6
        flops = 4 * B * H * S * S * D / 2
        results["sdpa_weights"] = {
            "workload": "bf16 causal SDPA with the attention weights returned (the math op) B=2 H=16 S=2048 D=128",
            "value": round(gbs, 1), "unit": "GB/s", "ms_per_step": round(ms, 4), "tflops_causal_halved": round(flops / ms / 1e9, 1),
            "kernel": "weights_fwd_kernel<bf16,128,causal>", "algorithmic_bytes_per_launch": nbytes,
            "roofline": roofline("hbm", gbs, "weights_fwd_kernel"),
        }
        log(f"sdpa_weights: {ms * 1e3:.1f} us  {gbs:.0f} GB/s ({gbs / HBM_PEAK_GBS:.1%})  {flops / ms / 1e9:.0f} TFLOP/s (causal-halved count)")
        w_got, o_got = attn[1, 5, :192, :192].cpu(), out[1, 5, :192].cpu()

        def check_weights(O, qc=qc, kc=kc, vc=vc, w_got=w_got, o_got=o_got, scale=scale):
            # a causal query sees its prefix only: the first 192 queries of a head stand alone
            ref_o, ref_w = O.sdpa_math(qc[1:2, 5:6, :192], kc[1:2, 5:6, :192], vc[1:2, 5:6, :192], is_causal=True, scale=scale, gemm="aten")
            diff = w_got.view(torch.int16).int() - ref_w[0, 0].view(torch.int16).int()
            off_by_more = int((diff.abs() > 1).sum())
            differing = int((diff != 0).sum())
            err_o = (o_got.float() - ref_o[0, 0].float()).abs().max().item()
            n = w_got.numel()
            return {"weights_differing": differing, "weights_off_by_more_than_one_ulp": off_by_more, "elements": n, "out_max_abs_err": err_o,
                    "tolerance": "weights: at most 5e-3 of the elements differ, 5e-4 by more than one ulp; out 2e-2",
                    "ok": differing <= 5e-3 * n and off_by_more <= 5e-4 * n and err_o <= 2e-2, "slice": "queries and keys 0..191 of head (1,5)"}
        checks["sdpa_weights"] = check_weights
        del q, k, v, out, attn

    # ------------------------------------------------------------------ configs[1]
    if want("rmsnorm_swiglu"):
        torch.manual_seed(0)
        rows, Hd, I = 16384, 4096, 14336
        nrot = 4                                  # 4 x 268 MB of RMSNorm traffic between reuses of a buffer
        xc = draw(rows, Hd)
        wc = draw(Hd, mean=1.0, std=0.02)
        xs = [xc.to(dev)] + [torch.roll(xc, 37 * (j + 1), 0).to(dev) for j in range(nrot - 1)]   # the same rows, shifted
        outs = [torch.empty_like(x) for x in xs]
        w = wc.to(dev)
        rstd = torch.empty(rows, dtype=torch.float32, device=dev)

        def rms(i):
            j = i % nrot
            must(L.paras_rms_norm_fwd(xs[j].data_ptr(), w.data_ptr(), outs[j].data_ptr(), rstd.data_ptr(), rows, Hd,
                                      1e-6, capi.BF16, st))
        ms_r, _ = timer.run(rms, steps, warmup, SETTLE_MS)
        bytes_r = 2 * rows * Hd * 2 + Hd * 2 + rows * 4
        gbs_r = bytes_r / ms_r / 1e6
        rms_got = outs[0][:256].cpu()
        del xs, outs
        gc_, uc = draw(rows, I), draw(rows, I)
        gate, up = gc_.to(dev), uc.to(dev)
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
        sw_got = so[rows - 128:].cpu()
        x_head, g_tail, u_tail = xc[:256].clone(), gc_[rows - 128:].clone(), uc[rows - 128:].clone()

        def check_rs(O, x_head=x_head, wc=wc, g_tail=g_tail, u_tail=u_tail, rms_got=rms_got, sw_got=sw_got):
            ref_r, _ = O.rms_norm(x_head, wc, 1e-6)
            ref_s = O.swiglu(g_tail, u_tail)
            bad = int((rms_got.view(torch.int16) != ref_r.view(torch.int16)).sum()) + \
                int((sw_got.view(torch.int16) != ref_s.view(torch.int16)).sum())
            return {"mismatching_elements": bad, "tolerance": "bit-exact", "ok": bad == 0,
                    "slice": "RMSNorm rows 0..255, SwiGLU rows 16256..16383"}
        checks["rmsnorm_swiglu"] = check_rs
        del gate, up, so, xc, gc_, uc

    # ------------------------------------------------------------------ configs[3]
    if want("sdpa_decode"):
        torch.manual_seed(0)
        B, Hq, Hkv, Lk, D = 64, 32, 8, 8192, 128
        qc = draw(B, Hq, 1, D)
        kc, vc = draw(B, Hkv, Lk, D), draw(B, Hkv, Lk, D)
        q, k, v = qc.to(dev), kc.to(dev), vc.to(dev)
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
        dec_got = out[[0, 63]].cpu()
        dq, dk, dv = qc[[0, 63]].clone(), kc[[0, 63]].clone(), vc[[0, 63]].clone()

        def check_decode(O, dq=dq, dk=dk, dv=dv, dec_got=dec_got):
            ref, _ = O.sdpa_math(dq, dk, dv, enable_gqa=True, gemm="aten")
            worst = (dec_got.float() - ref.float()).abs().max().item()
            return {"max_abs_err": worst, "tolerance": 2e-2, "ok": worst <= 2e-2, "slice": "sequences 0 and 63, all 32 heads"}
        checks["sdpa_decode"] = check_decode
        del q, k, v, out, ws, qc, kc, vc

    # ------------------------------------------------------------------ configs[4]
    if want("moe"):
        torch.manual_seed(0)
        T, Hd, E, kk, I = 8192, 4096, 8, 2, 14336
        lc, xc = draw(T, E), draw(T, Hd)
        wgc, wuc, wdc = draw(E, I, Hd, std=0.02), draw(E, I, Hd, std=0.02), draw(E, Hd, I, std=0.02)
        x, logits = xc.to(dev), lc.to(dev)
        wg, wu, wd = wgc.to(dev), wuc.to(dev), wdc.to(dev)
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
        ms_route, _ = timer.run(route, max(steps, 20), max(warmup, 5), SETTLE_MS)
        ms_ffn, _ = timer.run(ffn, msteps, mwarm, SETTLE_MFMA_MS)
        ms_all, _ = timer.run(lambda i: (route(i), ffn(i)), msteps, mwarm, SETTLE_MFMA_MS)
        flops = T * kk * 3 * 2 * Hd * I
        tf = flops / ms_ffn / 1e9
        results["moe"] = {
            "workload": "bf16 MoE layer T=8192 H=4096 E=8 top-2 I=14336: routing + grouped expert FFN (configs[4])",
            "value": round(T / ms_all * 1e3, 1), "unit": "tokens/s", "ms_per_step": round(ms_all, 4), "steps": msteps,
            "route_ms": round(ms_route, 4), "ffn_ms": round(ms_ffn, 4), "ffn_tflops": round(tf, 2),
            "kernel": "grouped_gemm_quad16_kernel<bf16> (gate-up+SwiGLU, down) + moe_combine_kernel",
            "algorithmic_flops_per_launch": flops, "roofline": roofline("mfma", tf, "grouped_gemm_quad16_kernel"),
        }
        log(f"moe: route {ms_route * 1e3:.1f} us, ffn {ms_ffn * 1e3:.1f} us = {tf:.1f} TFLOP/s ({tf / MFMA_BF16_PEAK_TFLOPS:.1%}), "
            f"layer {ms_all * 1e3:.1f} us = {T / ms_all * 1e3:.0f} tokens/s")
        route_got = [t.cpu() for t in (topi, topw, order, inv, counts, offsets)]
        sel = torch.arange(0, T, T // 16)[:16] + 3
        moe_got = out.cpu()[sel]

        def check_moe(O, lc=lc, xc=xc, wgc=wgc, wuc=wuc, wdc=wdc, sel=sel, kk=kk, route_got=route_got, moe_got=moe_got):
            want_r = O.moe_route(lc, kk)
            bad = sum(int((g.view(torch.int32) != w_.view(torch.int32)).sum()) if g.dtype == torch.float32 else int((g != w_).sum())
                      for g, w_ in zip(route_got, want_r))
            r = O.moe_route(lc[sel], kk)     # a token's output depends only on its own row and routing
            ref = O.moe_ffn(xc[sel], wgc, wuc, wdc, r[1], r[2], r[3], r[5], kk, gemm="aten")
            err = (moe_got.float() - ref.float()).abs()
            ulp = 2.0 ** (torch.floor(torch.log2(ref.float().abs().clamp_min(1e-30))) - 7)   # one bf16 ulp of the reference value
            beyond = int((err > 2e-2).sum())
            # the test suite's bar: at most 1e-3 of the elements beyond max(2e-2, 1 ulp), none beyond one ulp of the top binade
            frac = float((err > torch.maximum(torch.full_like(err, 2e-2), ulp * 1.001)).float().mean())
            top = 2.0 ** (math.floor(math.log2(max(ref.float().abs().max().item(), 1e-30) * 1.999)) - 7)
            ok = frac <= 1e-3 and err.max().item() <= max(2e-2, top) * 1.001
            return {"routing_mismatches": bad, "max_abs_err": err.max().item(), "elements_beyond_2e-2": beyond, "elements": err.numel(),
                    "max_abs_reference": ref.float().abs().max().item(),
                    "tolerance": "routing bit-exact; FFN max(2e-2, one bf16 ulp of the reference value) for all but 1e-3 of the elements, one ulp of the largest output for those",
                    "ok": bad == 0 and ok, "slice": "routing of all 8192 tokens; FFN output of 16 tokens"}
        checks["moe"] = check_moe
        del x, wg, wu, wd, fws, out

    # ------------------------------------------------------------------ dense projection (the callers either side of the path)
    if want("linear"):
        torch.manual_seed(0)
        M, N, K = 16384, 4096, 4096               # 4 x 4096 tokens through a hidden x hidden nn.Linear
        xac, wbc = draw(M, K), draw(N, K, std=0.02)
        xa, wb = xac.to(dev), wbc.to(dev)
        yc = torch.empty(M, N, dtype=bf, device=dev)
        ms, _ = timer.run(lambda i: must(L.paras_gemm_nt(xa.data_ptr(), wb.data_ptr(), None, yc.data_ptr(), M, N, K, K, K, N, 0,
                                                         1, 0, 0, 0, 0, 1.0, 0.0, capi.BF16, st)), steps, warmup, SETTLE_MFMA_MS)
        flops = 2 * M * N * K
        tf = flops / ms / 1e9
        results["linear"] = {
            "workload": "bf16 dense NT GEMM x W^T: M=16384 N=4096 K=4096 (nn.Linear of configs[2]'s tokens)",
            "value": round(tf, 2), "unit": "TFLOP/s", "ms_per_step": round(ms, 4), "kernel": "dense_gemm_nt_quad16_kernel<bf16>",
            "algorithmic_flops_per_launch": flops, "roofline": roofline("mfma", tf, "dense_gemm_nt_quad16_kernel"),
        }
        log(f"linear: {ms * 1e3:.1f} us  {tf:.1f} TFLOP/s ({tf / MFMA_BF16_PEAK_TFLOPS:.1%})")
        lin_got = yc[M - 64:].cpu()
        xa_tail = xac[M - 64:].clone()

        def check_linear(O, xa_tail=xa_tail, wbc=wbc, lin_got=lin_got):
            ref = O.matmul_nt(xa_tail, wbc, gemm="aten")
            err = (lin_got.float() - ref.float()).abs()
            ulp = 2.0 ** (torch.floor(torch.log2(ref.float().abs().clamp_min(2.0 ** -7))) - 7)   # one bf16 ulp, floored at 2^-14
            worst, ulps = err.max().item(), (err / ulp).max().item()
            return {"max_abs_err": worst, "max_err_ulps": ulps, "tolerance": "2e-2 absolute and one bf16 ulp (floored at 2^-14) of ATen-CPU's product",
                    "ok": worst <= 2e-2 and ulps <= 1.001, "slice": "rows 16320..16383"}
        checks["linear"] = check_linear
        del xa, wb, yc, xac

    # ------------------------------------------------------------------ the ops either side of the path
    if want("backward_ops"):
        torch.manual_seed(0)
        rows, Hd, I = 16384, 4096, 14336
        nrot = 3                                  # every buffer is out of the 256 MB last-level cache when it comes round again
        xc, goc = draw(rows, Hd), draw(rows, Hd)
        wc = draw(Hd, mean=1.0, std=0.02)
        xb = [xc.to(dev) for _ in range(nrot)]    # rstd belongs to x: every set holds the same rows at its own address
        gob = [goc.to(dev)] + [torch.roll(goc, 37 * (j + 1), 0).to(dev) for j in range(nrot - 1)]
        w = wc.to(dev)
        y, gw = torch.empty_like(xb[0]), torch.empty_like(w)
        gxb = [torch.empty_like(xb[0]) for _ in range(nrot)]
        rstd = torch.empty(rows, dtype=torch.float32, device=dev)
        must(L.paras_rms_norm_fwd(xb[0].data_ptr(), w.data_ptr(), y.data_ptr(), rstd.data_ptr(), rows, Hd, 1e-6, capi.BF16, st))
        ws = torch.empty(L.paras_rms_norm_bwd_workspace(rows, Hd), dtype=torch.uint8, device=dev)
        ms_b, _ = timer.run(lambda i: must(L.paras_rms_norm_bwd(gob[i % nrot].data_ptr(), xb[i % nrot].data_ptr(), w.data_ptr(),
                                                                 rstd.data_ptr(), gxb[i % nrot].data_ptr(), gw.data_ptr(),
                                                                 ws.data_ptr(), rows, Hd, capi.BF16, st)),
                            steps, warmup, SETTLE_MS)
        bytes_b = 3 * rows * Hd * 2 + rows * 4 + 2 * Hd * 2
        # one more launch on buffer set 0 so that grad_w belongs to the grad_out the check holds
        must(L.paras_rms_norm_bwd(gob[0].data_ptr(), xb[0].data_ptr(), w.data_ptr(), rstd.data_ptr(), gxb[0].data_ptr(),
                                  gw.data_ptr(), ws.data_ptr(), rows, Hd, capi.BF16, st))
        gx_got, gw_got, rstd_c = gxb[0][:128].cpu(), gw.cpu(), rstd.cpu()
        del y, gxb, xb, gob, ws
        gc_, uc, g2c = draw(rows, I), draw(rows, I), draw(rows, I)
        gate, up, g2 = gc_.to(dev), uc.to(dev), g2c.to(dev)
        dg, du = torch.empty_like(gate), torch.empty_like(gate)
        n = rows * I
        ms_s, _ = timer.run(lambda i: must(L.paras_swiglu_bwd(g2.data_ptr(), gate.data_ptr(), up.data_ptr(), dg.data_ptr(),
                                                               du.data_ptr(), n, capi.BF16, st)), steps, warmup, SETTLE_MS)
        bytes_s = 5 * n * 2
        dg_got, du_got = dg[:64].cpu(), du[:64].cpu()
        sb_in = (g2c[:64].clone(), gc_[:64].clone(), uc[:64].clone())
        del gate, up, g2, dg, du, gc_, uc, g2c
        qhc = draw(4 * 32 * 4096, 128)
        qhs = [qhc.to(dev)] + [torch.roll(qhc, 11 * (j + 1), 0).to(dev) for j in range(3)]
        qos = [torch.empty_like(q_) for q_ in qhs]
        qh = qhs[0]
        ms_r, _ = timer.run(lambda i: must(L.paras_rotate_half(qhs[i % 4].data_ptr(), qos[i % 4].data_ptr(), qh.shape[0], 128, 0,
                                                               capi.BF16, st)), steps, warmup, SETTLE_MS)
        bytes_r = 2 * qh.numel() * 2
        rh_got, rh_in = qos[0][:512].cpu(), qhc[:512].clone()
        gb = lambda b, ms: b / ms / 1e6
        results["backward_ops"] = {
            "workload": "bf16 RMSNorm backward 16384x4096, SwiGLU backward 16384x14336, rotate_half 4x32x4096x128",
            "value": round((bytes_b + bytes_s + bytes_r) / (ms_b + ms_s + ms_r) / 1e6, 1), "unit": "GB/s",
            "ms_per_step": round(ms_b + ms_s + ms_r, 4),
            "rms_norm_bwd": {"ms": round(ms_b, 4), "algorithmic_bytes_per_launch": bytes_b,
                             "kernel": "rms_norm_bwd_fused<bf16> + rms_norm_bwd_dw_final_wide",
                             "roofline": roofline("hbm", gb(bytes_b, ms_b), "rms_norm_bwd_fused")},
            "swiglu_bwd": {"ms": round(ms_s, 4), "algorithmic_bytes_per_launch": bytes_s, "kernel": "swiglu_bwd_vec<bf16>",
                           "roofline": roofline("hbm", gb(bytes_s, ms_s), "swiglu_bwd_vec")},
            "rotate_half": {"ms": round(ms_r, 4), "algorithmic_bytes_per_launch": bytes_r, "kernel": "rotate_half_vec16",
                            "roofline": roofline("hbm", gb(bytes_r, ms_r), "rotate_half_vec16")},
        }
        log(f"backward_ops: rms_norm_bwd {ms_b * 1e3:.1f} us {gb(bytes_b, ms_b):.0f} GB/s ({gb(bytes_b, ms_b) / HBM_PEAK_GBS:.1%})   "
            f"swiglu_bwd {ms_s * 1e3:.1f} us {gb(bytes_s, ms_s):.0f} GB/s ({gb(bytes_s, ms_s) / HBM_PEAK_GBS:.1%})   "
            f"rotate_half {ms_r * 1e3:.1f} us {gb(bytes_r, ms_r):.0f} GB/s ({gb(bytes_r, ms_r) / HBM_PEAK_GBS:.1%})")

        def check_bwd(O, goc=goc, xc=xc, wc=wc, rstd_c=rstd_c, gx_got=gx_got, gw_got=gw_got, sb_in=sb_in, dg_got=dg_got,
                      du_got=du_got, rh_got=rh_got, rh_in=rh_in):
            b16 = lambda t: t.contiguous().view(torch.int16)
            ref_gx, ref_gw = O.rms_norm_backward(goc, xc, wc, rstd_c)
            bad = int((b16(gx_got) != b16(ref_gx[:128])).sum()) + int((b16(gw_got) != b16(ref_gw)).sum())
            rg, ru = O.swiglu_backward(*sb_in)
            bad += int((b16(dg_got) != b16(rg)).sum()) + int((b16(du_got) != b16(ru)).sum())
            bad += int((b16(rh_got) != b16(O.rotate_half(rh_in))).sum())
            return {"mismatching_elements": bad, "tolerance": "bit-exact", "ok": bad == 0,
                    "slice": "grad_x rows 0..127 and all of grad_w; SwiGLU backward rows 0..63; rotate_half rows 0..511"}
        checks["backward_ops"] = check_bwd
        del qh, qhs, qos

    # ------------------------------------------------------------------ counter calibration
    if args.workload == "copy":
        n = 1 << 29                                # 2^29 bf16 elements: 1 GiB read + 1 GiB written
        src = torch.randn(n // 4096, 4096, device=dev).to(bf)
        dst = torch.empty_like(src)
        shape, stride = (C.c_int64 * 1)(n), (C.c_int64 * 1)(1)
        ms, _ = timer.run(lambda i: must(L.paras_copy_strided(src.data_ptr(), dst.data_ptr(), 1, shape, stride, stride, 2,
                                                              capi.BF16, capi.BF16, st)), steps, warmup, SETTLE_MS)
        gbs = 4 * n / ms / 1e6
        results["copy"] = {"workload": "plain device copy of 2^29 bf16 elements (counter calibration)", "value": round(gbs, 1),
                           "unit": "GB/s", "ms_per_step": round(ms, 4), "kernel": "copy kernel", "algorithmic_bytes_per_launch": 4 * n,
                           "roofline": roofline("hbm", gbs, "copy")}
        log(f"copy: {ms * 1e3:.1f} us  {gbs:.0f} GB/s ({gbs / HBM_PEAK_GBS:.1%})")

    # ------------------------------------------------------------------ cpu baseline + parity of what was timed
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    if not args.no_cpu:
        for name, res in results.items():
            base, parity = cpu_leg(name, checks.get(name))
            if base is not None:
                res["cpu_baseline"] = base
            res["parity_checked"] = parity is not None and "error" not in parity
            res["parity"] = parity
    else:
        for res in results.values():
            res["parity_checked"] = False

    head_name = "sdpa_prefill" if "sdpa_prefill" in results else next(iter(results))
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
                   "inputs": "torch.manual_seed(0), torch-CPU randn, moved to the device (resident in HBM before timing)",
                   "timing": f"HIP events on the launch stream around exactly `steps` launches, after `warmup` launches plus "
                             f"{SETTLE_MFMA_MS:.0f} ms (matrix kernels) / {SETTLE_MS:.0f} ms (streaming kernels) of untimed launches "
                             f"that let the clocks settle"},
        "roofline": head.get("roofline") or next(v["roofline"] for v in head.values() if isinstance(v, dict) and "roofline" in v),
        "cpu_baseline": head.get("cpu_baseline"),
        "parity_checked": head.get("parity_checked", False),
        "workloads": results,
    }
    if traffic.get("_stale"):
        line["traffic_measured_on_other_sources"] = True
    print(json.dumps(line))
    bad = [n_ for n_, r in results.items() if r.get("parity") and r["parity"].get("ok") is False]
    if bad:
        log(f"bench.py: the timed output of {bad} differs from the oracle beyond its tolerance")
        return 3
    return 0


# bounded CPU samples: shape, work of the sample in the workload's unit, unit, description
CPU_SAMPLES = {
    "sdpa_prefill": ({"B": 4, "H": 32, "S": 4096, "D": 128}, lambda s: 4 * s["B"] * s["H"] * s["S"] ** 2 * s["D"] / 2 / 1e12, "TFLOP/s",
                     "the whole workload once: B=4, H=32, S=4096, D=128"),
    "sdpa_weights": ({"B": 1, "H": 2, "S": 2048, "D": 128}, lambda s: (s["B"] * s["H"] * s["S"] ** 2 * 2 + 4 * s["B"] * s["H"] * s["S"] * s["D"] * 2) / 1e9, "GB/s",
                     "2 of the 32 heads (1/16 of the workload)"),
    "rmsnorm_swiglu": ({"rows": 16384, "H": 4096, "I": 14336}, lambda s: (2 * s["rows"] * s["H"] * 2 + 3 * s["rows"] * s["I"] * 2) / 1e9, "GB/s",
                       "the whole workload once: 16384 rows"),
    "sdpa_decode": ({"B": 32, "Hq": 32, "Hkv": 8, "Lk": 8192, "D": 128}, lambda s: 2 * s["B"] * s["Hkv"] * s["Lk"] * s["D"] * 2 / 1e9, "GB/s",
                    "B=32 of 64 sequences (1/2 of the workload)"),
    "moe": ({"T": 2048, "H": 4096, "E": 8, "k": 2, "I": 14336}, lambda s: s["T"] / 1.0, "tokens/s",
            "2048 of the 8192 tokens, all 8 experts' weights"),
    "linear": ({"M": 16384, "N": 4096, "K": 4096}, lambda s: 2 * s["M"] * s["N"] * s["K"] / 1e12, "TFLOP/s",
               "the whole workload once: M=16384, N=K=4096"),
    "backward_ops": ({"rows": 16384, "H": 4096, "I": 14336},
                     lambda s: (3 * s["rows"] * s["H"] * 2 + 5 * s["rows"] * s["I"] * 2 + 2 * 32 * s["rows"] * 128 * 2) / 1e9, "GB/s",
                     "the whole workload once: 16384 rows (rotate_half: 4*32*4096 rows of 128)"),
}


def cpu_leg(name: str, check):
    """The only place the oracle is touched: (1) times a bounded sample of the workload on the
    host cores -- the reference's own CPU flavor when oracle/_ref is present, else the oracle's
    restatement -- and (2) runs `check`, which compares a slice of the output the timed launches
    produced with the oracle.  Returns (cpu_baseline, parity); a failure of either part is
    reported in its object and never hides the GPU result."""
    import ref_engine as R
    base = None
    if name in CPU_SAMPLES:
        sample, work, unit, text = CPU_SAMPLES[name]
        try:
            if R.available():
                res = R.run("time_workload", name, sample)
                threads = R.run("host_threads")
                kind = "reference"
            else:
                res, threads, kind = port_baseline(name, sample)
            val = work(sample) / res["seconds"]
            log(f"cpu_baseline[{kind}] {name}: sample took {res['seconds']:.2f} s on {threads} threads -> {val:.4g} {unit}")
            base = {"value": float(f"{val:.4g}"), "unit": unit, "cores": threads, "kind": kind,
                    "sample": f"{text}; {res['seconds']:.2f} s of CPU work", "detail": res}
        except Exception as e:
            log(f"cpu_baseline {name} failed: {e}")
            base = {"value": None, "unit": unit, "cores": os.cpu_count(), "kind": "unavailable", "sample": str(e)[:200]}
    parity = None
    if check is not None:
        try:
            import oracle as O
            t0 = time.perf_counter()
            parity = check(O)
            parity["seconds"] = round(time.perf_counter() - t0, 2)
            log(f"parity {name}: {parity}")
        except Exception as e:
            log(f"parity check {name} failed to run: {e}")
            parity = {"error": str(e)[:200]}
    return base, parity


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
