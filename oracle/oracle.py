"""Python face of the CPU oracle (oracle/paras_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py; the product never imports it.

Tensors are torch CPU tensors used as typed byte containers; every arithmetic
step happens in the C restatement, except the GEMMs of the composed ops, which
can go either through the C double-accumulate GEMM (``gemm="c"``, small cases)
or through torch-CPU matmul (``gemm="aten"``) -- the library the reference
itself bounces its GEMMs to (csrc/ops/vision_ops.cpp:388-406).

The compositions restate, step by step with the reference's rounding points:
  sdpa_math            csrc/ops/attention_ops.cpp:71-136
  rms_norm_composed    csrc/ops/rms_swiglu_ops.cpp:43-75
  swiglu_composed      csrc/ops/rms_swiglu_ops.cpp:83-86
  moe_route / moe_ffn  the canonical MoE composition of reference primitives
                       (topk, _softmax, stable argsort, index_select, mm,
                       paras::swiglu, mul, sum)
"""
from __future__ import annotations

import ctypes as C
import math
import subprocess
import sys
from pathlib import Path

import torch

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "libparas_oracle.so"
_lib = None

F32, F16, BF16, F64 = 0, 1, 2, 3
_DT = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16, torch.float64: F64}
OP_ADD, OP_MUL, OP_DIV, OP_SUB = 0, 1, 2, 3
UN_POW, UN_RSQRT, UN_SILU, UN_SCALE = 0, 1, 2, 3


def build() -> Path:
    src = _HERE / "paras_oracle.c"
    subprocess.run(["gcc", "-O2", "-fPIC", "-shared", "-std=c11", "-fopenmp", "-ffp-contract=off",
                    "-o", str(_LIB_PATH), str(src), "-lm"], check=True)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            build()
        _lib = C.CDLL(str(_LIB_PATH))
        _lib.po_round_to_dtype.restype = C.c_double
        _lib.po_round_to_dtype.argtypes = [C.c_double, C.c_int]
        _lib.po_get_threads.restype = C.c_int
    return _lib


def set_threads(n: int) -> None:
    lib().po_set_threads(C.c_int(n))


def get_threads() -> int:
    return lib().po_get_threads()


def _p(t: torch.Tensor):
    assert t.device.type == "cpu" and t.is_contiguous(), "oracle wants contiguous CPU tensors"
    return C.c_void_p(t.data_ptr())


def _dt(t: torch.Tensor) -> int:
    return _DT[t.dtype]


def _l(v) -> C.c_long:
    return C.c_long(int(v))


def round_to_dtype(v: float, dtype: torch.dtype) -> float:
    return lib().po_round_to_dtype(C.c_double(v), _DT[dtype])


# ---------------------------------------------------------------------------
# fused ops
# ---------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float):
    """paras::rms_norm -> (out, rstd)   (csrc/ops/fused_ops.cpp:43-88)"""
    x = x.contiguous()
    w = w.contiguous()
    H = x.shape[-1]
    rows = x.numel() // H if H > 0 else 0
    assert w.numel() == H, "paras rms_norm: weight size must match the last dimension"
    out = torch.empty_like(x)
    rstd = torch.empty(rows, dtype=torch.float32)
    lib().po_rms_norm(_p(x), _p(w), _p(out), _p(rstd), _l(rows), _l(H), C.c_double(eps), _dt(x))
    return out, rstd


def rms_norm_backward(go, x, w, rstd):
    go, x, w = go.contiguous(), x.contiguous(), w.contiguous()
    H = x.shape[-1]
    rows = x.numel() // H if H > 0 else 0
    gx = torch.empty_like(x)
    gw = torch.zeros(H, dtype=w.dtype)
    lib().po_rms_norm_bwd(_p(go), _p(x), _p(w), _p(rstd.contiguous()), _p(gx), _p(gw), _l(rows), _l(H), _dt(x))
    return gx, gw


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """paras::swiglu(gate, up) = silu(gate) * up   (csrc/ops/fused_ops.cpp:162-194)"""
    assert gate.shape == up.shape, "paras swiglu: gate and up must have the same shape"
    gate, up = gate.contiguous(), up.contiguous()
    out = torch.empty_like(gate)
    lib().po_swiglu(_p(gate), _p(up), _p(out), _l(gate.numel()), _dt(gate))
    return out


def swiglu_backward(go, gate, up):
    go, gate, up = go.contiguous(), gate.contiguous(), up.contiguous()
    gg, gu = torch.empty_like(gate), torch.empty_like(up)
    lib().po_swiglu_bwd(_p(go), _p(gate), _p(up), _p(gg), _p(gu), _l(go.numel()), _dt(go))
    return gg, gu


def rotate_half(x: torch.Tensor, backward: bool = False) -> torch.Tensor:
    x = x.contiguous()
    D = x.shape[-1]
    out = torch.empty_like(x)
    if x.numel():
        lib().po_rotate_half(_p(x), _p(out), _l(x.numel() // D), _l(D), int(backward), _dt(x))
    return out


# ---------------------------------------------------------------------------
# primitives
# ---------------------------------------------------------------------------
def binary(op: int, a: torch.Tensor, b: torch.Tensor, alpha: float = 1.0) -> torch.Tensor:
    """Broadcasting elementwise op in the dtype of ``a`` (binary_kernel)."""
    shape = torch.broadcast_shapes(a.shape, b.shape)
    ae = a.expand(shape).contiguous()
    be = b.to(a.dtype).expand(shape).contiguous()
    out = torch.empty(shape, dtype=a.dtype)
    lib().po_binary(op, _p(ae), _p(be), _p(out), _l(out.numel()), C.c_double(alpha), _dt(a))
    return out


def binary_scalar(op: int, a: torch.Tensor, s: float, alpha: float = 1.0) -> torch.Tensor:
    a = a.contiguous()
    out = torch.empty_like(a)
    lib().po_binary_scalar(op, _p(a), C.c_double(s), _p(out), _l(a.numel()), C.c_double(alpha), _dt(a))
    return out


def unary(op: int, a: torch.Tensor, param: float = 0.0) -> torch.Tensor:
    a = a.contiguous()
    out = torch.empty_like(a)
    lib().po_unary(op, _p(a), _p(out), _l(a.numel()), C.c_double(param), _dt(a))
    return out


def softmax_last(x: torch.Tensor, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    x = x.contiguous()
    out = torch.empty(x.shape, dtype=out_dtype or x.dtype)
    n = x.shape[-1]
    if x.numel():
        lib().po_softmax_last(_p(x), _p(out), _l(x.numel() // n), _l(n), _dt(x), _dt(out))
    return out


def sum_last(x: torch.Tensor) -> torch.Tensor:
    x = x.contiguous()
    n = x.shape[-1]
    out = torch.empty(x.shape[:-1], dtype=x.dtype)
    lib().po_sum_last(_p(x), _p(out), _l(out.numel()), _l(n), _dt(x))
    return out


def sum_mid(x: torch.Tensor) -> torch.Tensor:
    """Sum over dim 1 of a contiguous [outer, red, inner] tensor."""
    x = x.contiguous()
    o, r, i = x.shape
    out = torch.empty(o, i, dtype=x.dtype)
    lib().po_sum_mid(_p(x), _p(out), _l(o), _l(r), _l(i), _dt(x))
    return out


def mean_last_keepdim(x: torch.Tensor, ndims: int = 1) -> torch.Tensor:
    """mean over the trailing ``ndims`` dims, keepdim: sum narrowed to the
    dtype, then a separate multiply by 1/count narrowed again
    (csrc/ops/pointwise_ops.cpp:776-787, 216-219)."""
    lead = x.shape[: x.dim() - ndims]
    count = 1
    for s in x.shape[x.dim() - ndims:]:
        count *= s
    s = sum_last(x.reshape(*lead, count))
    m = unary(UN_SCALE, s, 1.0 / count if count > 0 else 0.0)
    return m.reshape(*lead, *([1] * ndims))


def topk_last(x: torch.Tensor, k: int, largest: bool = True):
    x = x.contiguous()
    n = x.shape[-1]
    rows = x.numel() // n if n else 0
    vals = torch.empty(*x.shape[:-1], k, dtype=x.dtype)
    idx = torch.empty(*x.shape[:-1], k, dtype=torch.int64)
    lib().po_topk_last(_p(x), _l(rows), _l(n), _l(k), int(largest), _p(vals), _p(idx), _dt(x))
    return vals, idx


def argsort_stable(keys: torch.Tensor) -> torch.Tensor:
    keys = keys.contiguous()
    assert keys.dtype == torch.int64 and keys.dim() == 1
    out = torch.empty_like(keys)
    lib().po_argsort_stable_i64(_p(keys), _p(out), _l(keys.numel()))
    return out


def index_select_rows(src: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    src = src.contiguous()
    idx = idx.contiguous()
    row = src[0].numel() * src.element_size() if src.shape[0] else 0
    out = torch.empty(idx.numel(), *src.shape[1:], dtype=src.dtype)
    lib().po_index_select_rows(_p(src), _p(idx), _p(out), _l(idx.numel()), _l(row))
    return out


def matmul_nt(a: torch.Tensor, b: torch.Tensor, gemm: str = "c") -> torch.Tensor:
    """a[..., M, K] @ b[..., N, K]^T in the dtype of a, one rounding."""
    if gemm == "aten":
        return torch.matmul(a, b.transpose(-1, -2))
    a, b = a.contiguous(), b.contiguous()
    M, K = a.shape[-2:]
    N = b.shape[-2]
    batch = a.shape[:-2]
    out = torch.empty(*batch, M, N, dtype=a.dtype)
    a3, b3, o3 = a.reshape(-1, M, K), b.reshape(-1, N, K), out.reshape(-1, M, N)
    for i in range(a3.shape[0]):
        lib().po_matmul_nt(_p(a3[i]), _p(b3[i]), _p(o3[i]), _l(M), _l(N), _l(K), _dt(a))
    return out


def matmul_nn(a: torch.Tensor, b: torch.Tensor, gemm: str = "c") -> torch.Tensor:
    if gemm == "aten":
        return torch.matmul(a, b)
    a, b = a.contiguous(), b.contiguous()
    M, K = a.shape[-2:]
    N = b.shape[-1]
    batch = a.shape[:-2]
    out = torch.empty(*batch, M, N, dtype=a.dtype)
    a3, b3, o3 = a.reshape(-1, M, K), b.reshape(-1, K, N), out.reshape(-1, M, N)
    for i in range(a3.shape[0]):
        lib().po_matmul_nn(_p(a3[i]), _p(b3[i]), _p(o3[i]), _l(M), _l(N), _l(K), _dt(a))
    return out


# ---------------------------------------------------------------------------
# compositions
# ---------------------------------------------------------------------------
def sdpa_math(q, k, v, attn_mask=None, is_causal=False, scale=None, enable_gqa=False, gemm="c"):
    """aten::_scaled_dot_product_attention_math on the host engine
    (csrc/ops/attention_ops.cpp:71-136), dropout_p == 0.  Returns (out, attn)."""
    assert q.dim() >= 3 and k.dim() >= 3 and v.dim() >= 3
    assert not (is_causal and attn_mask is not None)
    if enable_gqa and k.shape[-3] != q.shape[-3]:
        assert q.shape[-3] % k.shape[-3] == 0
        rep = q.shape[-3] // k.shape[-3]
        k = k.repeat_interleave(rep, dim=-3)       # pure copy (tensor_ops.cpp:687-729)
        v = v.repeat_interleave(rep, dim=-3)
    D = q.shape[-1]
    scale_factor = scale if scale is not None else 1.0 / math.sqrt(float(D))
    bshape = torch.broadcast_shapes(q.shape[:-2], k.shape[:-2])
    qe = q.expand(*bshape, *q.shape[-2:])
    ke = k.expand(*bshape, *k.shape[-2:])
    ve = v.expand(*bshape, *v.shape[-2:])
    scores = matmul_nt(qe, ke, gemm)                          # at::matmul -> bmm, rounded to dtype
    scores = binary_scalar(OP_MUL, scores, scale_factor)      # scalar narrowed to dtype first
    Lq, Lk = q.shape[-2], k.shape[-2]
    if is_causal:
        allow = torch.empty(Lq, Lk, dtype=torch.uint8)
        lib().po_tril_ones(_p(allow), _l(Lq), _l(Lk), _l(0))
        deny = (allow == 0).to(torch.uint8).expand(scores.shape).contiguous()
        lib().po_masked_fill(_p(scores), _p(deny), C.c_double(-math.inf), _l(scores.numel()), _dt(scores))
    elif attn_mask is not None:
        if attn_mask.dtype == torch.bool:
            deny = (~attn_mask).to(torch.uint8).expand(scores.shape).contiguous()
            lib().po_masked_fill(_p(scores), _p(deny), C.c_double(-math.inf), _l(scores.numel()), _dt(scores))
        else:
            scores = binary(OP_ADD, scores, attn_mask, 1.0)
    attn = softmax_last(scores)
    out = matmul_nn(attn, ve, gemm)
    return out, attn


def rms_norm_composed(x, normalized_shape, weight=None, eps=None):
    """aten::rms_norm on the host engine (csrc/ops/rms_swiglu_ops.cpp:43-75):
    pow(2) -> mean(keepdim) -> + eps -> rsqrt -> x * inv -> * weight, each
    step narrowed to the tensor dtype."""
    nd = len(normalized_shape)
    assert nd >= 1 and x.dim() >= nd and tuple(x.shape[-nd:]) == tuple(normalized_shape)
    eps_val = 1e-6 if eps is None else eps
    ms = mean_last_keepdim(unary(UN_POW, x, 2.0), nd)
    inv = unary(UN_RSQRT, binary_scalar(OP_ADD, ms, eps_val, 1.0))
    out = binary(OP_MUL, x, inv)
    if weight is not None:
        assert tuple(weight.shape) == tuple(normalized_shape)
        out = binary(OP_MUL, out, weight)
    return out


def swiglu_composed(x, gate):
    """torch_paras::swiglu(x, gate) = x * silu(gate) (rms_swiglu_ops.cpp:83-86)."""
    return binary(OP_MUL, x, unary(UN_SILU, gate))


def moe_route(logits: torch.Tensor, k: int):
    """topk -> softmax of the kept logits in fp32 -> stable expert-major order.
    Returns (topi[T,k] i64, topw[T,k] f32, order[T*k] i64, inv_order[T*k] i64,
    counts[E] i64, offsets[E+1] i64)."""
    T, E = logits.shape
    topv, topi = topk_last(logits, k, True)
    topw = softmax_last(topv.float())
    flat_e = topi.reshape(-1)
    order = argsort_stable(flat_e)
    inv = argsort_stable(order)
    counts = torch.bincount(flat_e, minlength=E).to(torch.int64)
    offsets = torch.zeros(E + 1, dtype=torch.int64)
    offsets[1:] = torch.cumsum(counts, 0)
    return topi, topw, order, inv, counts, offsets


def moe_ffn(x, w_gate, w_up, w_down, topw, order, inv_order, offsets, k, gemm="c"):
    """Grouped expert FFN + weighted combine; every GEMM result, the SwiGLU,
    the weighting and the slot sum are each narrowed to the tensor dtype."""
    T, H = x.shape
    E = w_gate.shape[0]
    xp = index_select_rows(x, order // k)
    y = torch.empty(T * k, H, dtype=x.dtype)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi == lo:
            continue
        g = matmul_nt(xp[lo:hi], w_gate[e], gemm)
        u = matmul_nt(xp[lo:hi], w_up[e], gemm)
        h = swiglu(g, u)
        y[lo:hi] = matmul_nt(h, w_down[e], gemm)
    yt = index_select_rows(y, inv_order).reshape(T, k, H)
    wt = topw.to(x.dtype).reshape(T, k, 1)
    return sum_mid(binary(OP_MUL, yt, wt))


def main(argv):
    if argv and argv[0] == "build":
        print(build())


if __name__ == "__main__":
    main(sys.argv[1:])
