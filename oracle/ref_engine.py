"""Loader for oracle/_ref/libparas_ref.so -- the reference's own CPU flavor
(its `paras:0` host engine), compiled from the reference sources by
oracle/Makefile.ref.

TEST INFRASTRUCTURE ONLY.  It validates the C restatement (oracle/paras_oracle.c)
and serves as bench.py's timed CPU baseline (cpu_baseline.kind == "reference").

The library claims PyTorch's PrivateUse1 device for itself, and so does the
product's torch_paras package; one process can hold only one of them.  Use
``load()`` in a process that has not imported torch_paras, or ``run()`` to
evaluate a function in a child process.

Only the compiled C++ is used: the reference's Python package is not imported;
the few lines below register the device module PyTorch wants for a renamed
PrivateUse1 backend.
"""
from __future__ import annotations

import os
import subprocess
import sys
import tempfile
import types
from pathlib import Path

import torch

_HERE = Path(__file__).resolve().parent
LIB = _HERE / "_ref" / "libparas_ref.so"
DEVICE = "paras:0"
_loaded = False


def available() -> bool:
    return LIB.exists()


def load() -> None:
    """Registers the reference engine as device `paras` in this process."""
    global _loaded
    if _loaded:
        return
    if "torch_paras" in sys.modules:
        raise RuntimeError("the product's torch_paras already owns PrivateUse1 in this process")
    torch.ops.load_library(str(LIB))
    torch.utils.rename_privateuse1_backend("paras")
    mod = types.ModuleType("torch.paras")
    mod.device_count = lambda: 1
    mod.is_available = lambda: True
    mod.current_device = lambda: 0
    mod.is_bad_fork = lambda: False
    mod._is_in_bad_fork = lambda: False
    mod.manual_seed_all = lambda seed: None
    mod.get_amp_supported_dtype = lambda: [torch.float16, torch.float32]
    torch._register_device_module("paras", mod)
    _loaded = True


# --- functions evaluated on the reference engine (inputs/outputs: CPU tensors) ---
def _dev(t):
    return t.to(DEVICE) if torch.is_tensor(t) else t


def _cpu(x):
    if torch.is_tensor(x):
        return x.cpu()
    if isinstance(x, (tuple, list)):
        return tuple(_cpu(i) for i in x)
    return x


def rms_norm(x, w, eps):
    return _cpu(torch.ops.paras.rms_norm(_dev(x), _dev(w), eps))


def rms_norm_backward(go, x, w, rstd):
    return _cpu(torch.ops.paras.rms_norm_backward(_dev(go), _dev(x), _dev(w), _dev(rstd)))


def swiglu(gate, up):
    return _cpu(torch.ops.paras.swiglu(_dev(gate), _dev(up)))


def swiglu_backward(go, gate, up):
    return _cpu(torch.ops.paras.swiglu_backward(_dev(go), _dev(gate), _dev(up)))


def rotate_half(x, backward=False):
    fn = torch.ops.paras.rotate_half_backward if backward else torch.ops.paras.rotate_half
    return _cpu(fn(_dev(x)))


def rms_norm_composed(x, normalized_shape, weight=None, eps=None):
    return _cpu(torch.ops.aten.rms_norm(_dev(x), list(normalized_shape), _dev(weight), eps))


def swiglu_composed(x, gate):
    return _cpu(torch.ops.torch_paras.swiglu(_dev(x), _dev(gate)))


def sdpa_math(q, k, v, attn_mask=None, is_causal=False, scale=None, enable_gqa=False):
    return _cpu(torch.ops.aten._scaled_dot_product_attention_math(
        _dev(q), _dev(k), _dev(v), _dev(attn_mask), 0.0, is_causal, None, scale=scale, enable_gqa=enable_gqa))


def softmax_last(x, out_dtype=None):
    half_to_float = out_dtype is not None and out_dtype != x.dtype
    return _cpu(torch.ops.aten._softmax(_dev(x), -1, half_to_float))


def topk_last(x, k, largest=True):
    return _cpu(torch.topk(_dev(x), k, dim=-1, largest=largest, sorted=True))


def argsort_stable(keys):
    return _cpu(torch.argsort(_dev(keys), dim=-1, stable=True))


def binary(op, a, b, alpha=1.0):
    """add / mul / div / sub (the oracle's op codes 0..3) of two tensors (binary_kernel,
    csrc/ops/pointwise_ops.cpp:62-85,262-302); alpha scales b for add and sub."""
    da, db = _dev(a), _dev(b)
    if op == 0:
        return _cpu(torch.add(da, db, alpha=alpha))
    if op == 3:
        return _cpu(torch.sub(da, db, alpha=alpha))
    return _cpu(torch.mul(da, db) if op == 1 else torch.div(da, db))


def binary_scalar(op, a, s, alpha=1.0):
    """The same ops with a Python number as the second operand (narrowed to the tensor type first)."""
    da = _dev(a)
    if op == 0:
        return _cpu(torch.add(da, s, alpha=alpha))
    if op == 3:
        return _cpu(torch.sub(da, s, alpha=alpha))
    return _cpu(torch.mul(da, s) if op == 1 else torch.div(da, s))


def index_select_rows(src, idx):
    return _cpu(torch.index_select(_dev(src), 0, _dev(idx)))


def moe_route(logits, k):
    """The canonical MoE routing composition, each step on the reference engine."""
    d = _dev(logits)
    T, E = logits.shape
    topv, topi = torch.topk(d, k, dim=-1)
    topw = torch.ops.aten._softmax(topv.float(), -1, False)
    flat_e = topi.reshape(-1)
    order = torch.argsort(flat_e, dim=-1, stable=True)
    inv = torch.argsort(order, dim=-1, stable=True)
    flat_cpu = flat_e.cpu()
    counts = torch.bincount(flat_cpu, minlength=E).to(torch.int64)
    offsets = torch.zeros(E + 1, dtype=torch.int64)
    offsets[1:] = torch.cumsum(counts, 0)
    return topi.cpu(), topw.cpu(), order.cpu(), inv.cpu(), counts, offsets


def moe_ffn(x, w_gate, w_up, w_down, topw, order, inv_order, offsets, k):
    T, H = x.shape
    E = w_gate.shape[0]
    dx = _dev(x)
    xp = torch.index_select(dx, 0, _dev(order // k))
    ys = []
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi == lo:
            continue
        rows = xp[lo:hi]
        g = torch.mm(rows, _dev(w_gate[e]).t())
        u = torch.mm(rows, _dev(w_up[e]).t())
        h = torch.ops.paras.swiglu(g, u)
        ys.append(torch.mm(h, _dev(w_down[e]).t()))
    y = torch.cat([t.cpu() for t in ys], 0).to(DEVICE)
    yt = torch.index_select(y, 0, _dev(inv_order)).reshape(T, k, H)
    wt = _dev(topw).to(x.dtype).reshape(T, k, 1)
    return (yt * wt).sum(1).cpu()


# --- timed samples for bench.py's cpu_baseline leg (run in a child process) --------
def time_workload(name: str, sample: dict) -> dict:
    """Builds seeded inputs of the sampled shape, runs the workload once on the
    reference engine (after one small warm-up call), returns wall seconds."""
    import time
    torch.manual_seed(0)
    bf = torch.bfloat16
    if name == "sdpa_prefill":
        B, H, S, D = sample["B"], sample["H"], sample["S"], sample["D"]
        q, k, v = (torch.randn(B, H, S, D).to(bf) for _ in range(3))
        sdpa_math(q[:, :1, :64], k[:, :1, :64], v[:, :1, :64], is_causal=True)
        dq, dk, dv = _dev(q), _dev(k), _dev(v)
        t0 = time.perf_counter()
        out = torch.ops.aten._scaled_dot_product_attention_math(dq, dk, dv, None, 0.0, True, None, scale=None, enable_gqa=False)[0]
        out.cpu()
        return {"seconds": time.perf_counter() - t0}
    if name == "sdpa_weights":
        B, H, S, D = sample["B"], sample["H"], sample["S"], sample["D"]
        q, k, v = (torch.randn(B, H, S, D).to(bf) for _ in range(3))
        sdpa_math(q[:, :1, :64], k[:, :1, :64], v[:, :1, :64], is_causal=True)
        dq, dk, dv = _dev(q), _dev(k), _dev(v)
        t0 = time.perf_counter()
        out, attn = torch.ops.aten._scaled_dot_product_attention_math(dq, dk, dv, None, 0.0, True, None, scale=None, enable_gqa=False)
        out.cpu()
        attn.cpu()
        return {"seconds": time.perf_counter() - t0}
    if name == "rmsnorm_swiglu":
        rows, H, I = sample["rows"], sample["H"], sample["I"]
        x, w = torch.randn(rows, H).to(bf), (1 + 0.02 * torch.randn(H)).to(bf)
        gate, up = torch.randn(rows, I).to(bf), torch.randn(rows, I).to(bf)
        rms_norm(x[:4], w, 1e-6)
        dx, dw, dg, du = _dev(x), _dev(w), _dev(gate), _dev(up)
        t0 = time.perf_counter()
        torch.ops.paras.rms_norm(dx, dw, 1e-6)
        t1 = time.perf_counter()
        torch.ops.paras.swiglu(dg, du)
        t2 = time.perf_counter()
        return {"seconds": t2 - t0, "rms_norm_seconds": t1 - t0, "swiglu_seconds": t2 - t1}
    if name == "sdpa_decode":
        B, Hq, Hkv, Lk, D = sample["B"], sample["Hq"], sample["Hkv"], sample["Lk"], sample["D"]
        q, k, v = torch.randn(B, Hq, 1, D).to(bf), torch.randn(B, Hkv, Lk, D).to(bf), torch.randn(B, Hkv, Lk, D).to(bf)
        dq, dk, dv = _dev(q), _dev(k), _dev(v)
        t0 = time.perf_counter()
        torch.ops.aten._scaled_dot_product_attention_math(dq, dk, dv, None, 0.0, False, None, scale=None, enable_gqa=True)[0].cpu()
        return {"seconds": time.perf_counter() - t0}
    if name == "moe":
        T, H, E, k, I = sample["T"], sample["H"], sample["E"], sample["k"], sample["I"]
        x, logits = torch.randn(T, H).to(bf), torch.randn(T, E).to(bf)
        wg, wu = (0.02 * torch.randn(E, I, H)).to(bf), (0.02 * torch.randn(E, I, H)).to(bf)
        wd = (0.02 * torch.randn(E, H, I)).to(bf)
        t0 = time.perf_counter()
        topi, topw, order, inv, counts, offsets = moe_route(logits, k)
        moe_ffn(x, wg, wu, wd, topw, order, inv, offsets, k)
        return {"seconds": time.perf_counter() - t0}
    if name == "linear":
        M, N, K = sample["M"], sample["N"], sample["K"]
        a, w = torch.randn(M, K).to(bf), (0.02 * torch.randn(N, K)).to(bf)
        da, dw = _dev(a), _dev(w)
        t0 = time.perf_counter()
        torch.mm(da, dw.t()).cpu()
        return {"seconds": time.perf_counter() - t0}
    if name == "backward_ops":
        rows, H, I = sample["rows"], sample["H"], sample["I"]
        x, go, w = torch.randn(rows, H).to(bf), torch.randn(rows, H).to(bf), (1 + 0.02 * torch.randn(H)).to(bf)
        gate, up, g2 = torch.randn(rows, I).to(bf), torch.randn(rows, I).to(bf), torch.randn(rows, I).to(bf)
        qh = torch.randn(32 * rows, 128).to(bf)
        dx, dgo, dw = _dev(x), _dev(go), _dev(w)
        rstd = torch.ops.paras.rms_norm(dx, dw, 1e-6)[1]
        dgate, dup, dg2, dqh = _dev(gate), _dev(up), _dev(g2), _dev(qh)
        t0 = time.perf_counter()
        torch.ops.paras.rms_norm_backward(dgo, dx, dw, rstd)
        t1 = time.perf_counter()
        torch.ops.paras.swiglu_backward(dg2, dgate, dup)
        t2 = time.perf_counter()
        torch.ops.paras.rotate_half(dqh)
        t3 = time.perf_counter()
        return {"seconds": t3 - t0, "rms_norm_bwd_seconds": t1 - t0, "swiglu_bwd_seconds": t2 - t1, "rotate_half_seconds": t3 - t2}
    raise ValueError(name)


def host_threads() -> int:
    """Threads the reference's host pool uses (csrc/compat/paras_compat.cpp:70-82)."""
    env = os.environ.get("PTSYCL_CPU_THREADS")
    return int(env) if env and int(env) > 0 else torch.get_num_threads()


# --- child-process evaluation ----------------------------------------------------
def run(fn_name: str, *args, threads: int | None = None, **kwargs):
    """Evaluates ``ref_engine.<fn_name>(*args, **kwargs)`` in a child process and
    returns its result (CPU tensors travel through a temporary file written
    and read by this module only)."""
    with tempfile.TemporaryDirectory() as td:
        inp, outp = Path(td) / "in.pt", Path(td) / "out.pt"
        torch.save({"fn": fn_name, "args": args, "kwargs": kwargs}, inp)
        env = dict(os.environ)
        if threads:
            env["PTSYCL_CPU_THREADS"] = str(threads)
            env["OMP_NUM_THREADS"] = str(threads)
        proc = subprocess.run([sys.executable, str(Path(__file__).resolve()), str(inp), str(outp)],
                              capture_output=True, text=True, env=env)
        if proc.returncode != 0:
            raise RuntimeError(f"reference engine failed:\n{proc.stdout}\n{proc.stderr}")
        return torch.load(outp, weights_only=False)


def run_batch(jobs, threads: int | None = None):
    """jobs: list of (fn_name, args, kwargs); one child process evaluates them
    all and the list of results comes back in the same order."""
    return run("_batch", jobs, threads=threads)


def _batch(jobs):
    return [globals()[name](*args, **kwargs) for name, args, kwargs in jobs]


def _child(inp: str, outp: str) -> None:
    load()
    req = torch.load(inp, weights_only=False)
    fn = globals()[req["fn"]]
    torch.save(fn(*req["args"], **req["kwargs"]), outp)


if __name__ == "__main__":
    _child(sys.argv[1], sys.argv[2])
