"""Writes tests/golden/hotpath.safetensors: inputs and expected outputs of the
hot-path functions, produced by the reference's own CPU flavor (its compiled
C++ host engine, oracle/_ref -- built by oracle/Makefile.ref from the
reference sources).  Run once in the authoring container:

    python tests/golden/make_golden.py

The file holds data only (tensors, named `<case>/<role>`), loaded with
safetensors.  Cases are small on purpose; they cover the dtypes, the mask /
causal / GQA variants, ties in routing, and ragged sizes.
"""
import math
import sys
from pathlib import Path

import torch
from safetensors.torch import save_file

ROOT = Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT / "oracle"))
import ref_engine as R  # noqa: E402


def main():
    R.load()
    g = torch.Generator().manual_seed(0)
    rn = lambda *s: torch.randn(*s, generator=g)
    out = {}

    def put(case, **tensors):
        for k, v in tensors.items():
            out[f"{case}/{k}"] = v.contiguous().clone()

    for name, dt in (("f32", torch.float32), ("bf16", torch.bfloat16), ("f16", torch.float16)):
        x, w, go = rn(9, 264).to(dt), (1 + 0.02 * rn(264)).to(dt), rn(9, 264).to(dt)
        o, rstd = R.rms_norm(x, w, 1e-6)
        gx, gw = R.rms_norm_backward(go, x, w, rstd)
        put(f"rms_norm_{name}", x=x, w=w, go=go, out=o, rstd=rstd, gx=gx, gw=gw)
        gate, up, gs = (3 * rn(5, 123)).to(dt), rn(5, 123).to(dt), rn(5, 123).to(dt)
        gg, gu = R.swiglu_backward(gs, gate, up)
        put(f"swiglu_{name}", gate=gate, up=up, go=gs, out=R.swiglu(gate, up), ggate=gg, gup=gu)
        put(f"rotate_half_{name}", x=x, out=R.rotate_half(x), bwd=R.rotate_half(x, True))
        put(f"rms_composed_{name}", x=x, w=w, out=R.rms_norm_composed(x, [264], w, 1e-5),
            out_now=R.rms_norm_composed(x, [264]))
        put(f"swiglu_composed_{name}", x=up, gate=gate, out=R.swiglu_composed(up, gate))

        q, k, v = rn(2, 4, 6, 16).to(dt), rn(2, 4, 10, 16).to(dt), rn(2, 4, 10, 16).to(dt)
        kg, vg = rn(2, 2, 10, 16).to(dt), rn(2, 2, 10, 16).to(dt)
        mask = torch.rand(2, 4, 6, 10, generator=g) > 0.3
        bias = (0.1 * rn(2, 4, 6, 10)).to(dt)
        put(f"sdpa_{name}", q=q, k=k, v=v, kg=kg, vg=vg, mask=mask.to(torch.uint8), bias=bias)
        for tag, kw in (("plain", {}), ("causal", dict(is_causal=True)), ("bool", dict(attn_mask=mask)),
                        ("bias", dict(attn_mask=bias)), ("scale", dict(scale=1 / math.sqrt(32)))):
            o, a = R.sdpa_math(q, k, v, **kw)
            put(f"sdpa_{name}", **{f"out_{tag}": o, f"attn_{tag}": a})
        o, a = R.sdpa_math(q, kg, vg, enable_gqa=True)
        put(f"sdpa_{name}", out_gqa=o, attn_gqa=a)

        logits = rn(70, 8).to(dt)
        logits[5] = logits[5, 0]
        logits[9, 3] = logits[9, 6]
        topi, topw, order, inv, counts, offsets = R.moe_route(logits, 2)
        put(f"moe_route_{name}", logits=logits, topi=topi, topw=topw, order=order, inv=inv, counts=counts,
            offsets=offsets)

    # flash-sized heads (D = 64 / 128) in bf16 / f16, causal with Lq != Lk and GQA
    for name, dt in (("bf16", torch.bfloat16), ("f16", torch.float16)):
        q, k, v = rn(1, 4, 40, 128).to(dt), rn(1, 2, 70, 128).to(dt), rn(1, 2, 70, 128).to(dt)
        put(f"sdpa_d128_{name}", q=q, k=k, v=v,
            out_causal=R.sdpa_math(q, k, v, is_causal=True, enable_gqa=True)[0],
            out_plain=R.sdpa_math(q, k, v, enable_gqa=True)[0])
        q1 = rn(1, 8, 1, 128).to(dt)   # decode: one query, 4 query heads per KV head, K/V shared with the case above
        put(f"sdpa_decode_{name}", q=q1, out=R.sdpa_math(q1, k, v, enable_gqa=True)[0])

    # MoE expert FFN (bf16, sizes the MFMA kernel accepts: multiples of 64)
    dt = torch.bfloat16
    T, E, kk, H, I = 40, 3, 2, 64, 64
    x, logits = rn(T, H).to(dt), rn(T, E).to(dt)
    wg, wu, wd = (0.1 * rn(E, I, H)).to(dt), (0.1 * rn(E, I, H)).to(dt), (0.1 * rn(E, H, I)).to(dt)
    topi, topw, order, inv, counts, offsets = R.moe_route(logits, kk)
    put("moe_ffn_bf16", x=x, logits=logits, wg=wg, wu=wu, wd=wd, topi=topi, topw=topw, order=order, inv=inv,
        offsets=offsets, out=R.moe_ffn(x, wg, wu, wd, topw, order, inv, offsets, kk))

    # the literals the reference's own tests hold
    t = torch.tensor([[5., 3., 5., 5., 1., 3.]])
    vals, idx = R.topk_last(t, 4)
    put("topk_ties_literal", x=t, vals=vals, idx=idx)
    put("argsort_literal", x=torch.tensor([3, 1, 2, 1, 3]), out=R.argsort_stable(torch.tensor([3, 1, 2, 1, 3])))

    # the glue primitives (drawn after everything above, so that the cases above keep their values)
    for name, dt in (("f32", torch.float32), ("bf16", torch.bfloat16), ("f16", torch.float16)):
        a, b, row = rn(6, 70).to(dt), (rn(6, 70) + 2.5).to(dt), rn(70).to(dt)
        idx = torch.tensor([5, 0, 0, 3, 2, 5, 1])
        put(f"glue_{name}", a=a, b=b, row=row, idx=idx,
            add=R.binary(0, a, b, 1.0), add_alpha=R.binary(0, a, b, -0.75), sub=R.binary(3, a, b, 1.0),
            sub_row_alpha=R.binary(3, a, row, 2.5), mul_row=R.binary(1, a, row), div=R.binary(2, a, b),
            add_s=R.binary_scalar(0, a, 0.3, 1.0), sub_s_alpha=R.binary_scalar(3, a, 0.3, 2.0),
            mul_s=R.binary_scalar(1, a, 1 / math.sqrt(128)), div_s=R.binary_scalar(2, a, 3.0),
            rows=R.index_select_rows(a, idx))

    path = Path(__file__).resolve().parent / "hotpath.safetensors"
    save_file(out, str(path))
    print(f"wrote {path} ({path.stat().st_size / 1024:.0f} KiB, {len(out)} tensors)")


if __name__ == "__main__":
    main()
