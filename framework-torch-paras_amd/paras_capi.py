"""ctypes binding of libparas_hip.so (the C ABI in include/paras_hip.h), as a
non-torch host would bind it.  torch CUDA tensors serve only as device memory
and a stream to launch on; the pointers handed over are plain HBM addresses.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import torch

PKG = Path(__file__).resolve().parent
LIB_PATH = PKG / "torch_paras" / "lib" / "libparas_hip.so"

F32, F16, BF16, F64 = 0, 1, 2, 3
DT = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16, torch.float64: F64}

i64, vp, f64, i32, sz = C.c_int64, C.c_void_p, C.c_double, C.c_int, C.c_size_t


class SdpaArgs(C.Structure):
    _fields_ = [
        ("q", vp), ("k", vp), ("v", vp), ("out", vp), ("attn", vp), ("lse", vp), ("mask", vp),
        ("mask_kind", C.c_int32), ("is_causal", C.c_int32), ("dtype", C.c_int32), ("reserved", C.c_int32),
        ("B", i64), ("Hq", i64), ("Hkv", i64), ("Lq", i64), ("Lk", i64), ("D", i64), ("Dv", i64),
        ("q_strides", i64 * 3), ("k_strides", i64 * 3), ("v_strides", i64 * 3), ("mask_strides", i64 * 4),
        ("scale", f64),
    ]


# name -> (restype, argtypes); the list is also what the symbol-export test walks.
SIGNATURES = {
    "paras_last_error": (C.c_char_p, []),
    "paras_abi_version": (i32, []),
    "paras_device_count": (i32, []),
    "paras_device_name": (i32, [i32, C.c_char_p, sz]),
    "paras_device_info": (i32, [i32, C.POINTER(i32), C.POINTER(C.c_uint64)]),
    "paras_stream": (i32, [i32, C.POINTER(vp)]),
    "paras_is_bad_fork": (i32, []),
    "paras_synchronize": (i32, [i32]),
    "paras_alloc": (i32, [i32, sz, C.POINTER(vp)]),
    "paras_free": (i32, [i32, vp]),
    "paras_empty_cache": (i32, [i32]),
    "paras_memory_stats": (i32, [i32, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "paras_round_size": (sz, [sz]),
    "paras_memcpy": (i32, [i32, vp, vp, sz, i32]),
    "paras_memset": (i32, [i32, vp, i32, sz]),
    "paras_copy_strided": (i32, [vp, vp, i32, C.POINTER(i64), C.POINTER(i64), C.POINTER(i64), i32, i32, i32, vp]),
    "paras_fill_strided": (i32, [vp, i32, C.POINTER(i64), C.POINTER(i64), i32, C.c_uint64, vp]),
    "paras_rms_norm_composed_fwd": (i32, [vp, vp, vp, i64, i64, f64, i32, vp]),
    "paras_swiglu_composed_fwd": (i32, [vp, vp, vp, i64, i32, vp]),
    "paras_rms_norm_fwd": (i32, [vp, vp, vp, vp, i64, i64, f64, i32, vp]),
    "paras_rms_norm_bwd_workspace": (sz, [i64, i64]),
    "paras_rms_norm_bwd": (i32, [vp, vp, vp, vp, vp, vp, vp, i64, i64, i32, vp]),
    "paras_swiglu_fwd": (i32, [vp, vp, vp, i64, i32, vp]),
    "paras_swiglu_bwd": (i32, [vp, vp, vp, vp, vp, i64, i32, vp]),
    "paras_rotate_half": (i32, [vp, vp, i64, i64, i32, i32, vp]),
    "paras_sdpa_workspace": (sz, [C.POINTER(SdpaArgs)]),
    "paras_sdpa_fwd": (i32, [C.POINTER(SdpaArgs), vp, vp]),
    "paras_sdpa_kernel_name": (C.c_char_p, [C.POINTER(SdpaArgs)]),
    "paras_moe_route_workspace": (sz, [i64, i64, i64]),
    "paras_moe_route": (i32, [vp, i64, i64, i64, i32, vp, vp, vp, vp, vp, vp, vp, vp]),
    "paras_moe_route_noalloc": (i32, [vp, i64, i64, i64, i32, vp, vp, vp, vp, vp, vp, vp]),
    "paras_moe_route_give_ups": (i32, [C.POINTER(C.c_uint64)]),
    "paras_mfma_rate_probe": (i32, [i32, i32, C.POINTER(C.c_double)]),
    "paras_l2_stream_probe": (i32, [i32, i32, C.POINTER(C.c_double)]),
    "paras_moe_ffn_workspace": (sz, [i64, i64, i64, i64, i32]),
    "paras_moe_ffn": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i32, vp]),
    "paras_index_select": (i32, [vp, vp, vp, i64, i64, i64, i64, vp]),
    "paras_binary_strided": (i32, [i32, vp, vp, vp, i32, vp, vp, vp, f64, i32, vp]),
    "paras_gemm_nt": (i32, [vp, vp, vp, vp] + [i64] * 12 + [f64, f64, i32, vp]),
    "paras_gemm_nt_workspace": (sz, [i64, i64, i64, i64, i32]),
    "paras_gemm_nt_ws": (i32, [vp, vp, vp, vp] + [i64] * 12 + [f64, f64, i32, vp, sz, vp]),
    "paras_softmax_rows": (i32, [vp, vp, i64, i64, i32, i32, vp]),
    "paras_topk_rows": (i32, [vp, vp, vp, i64, i64, i64, i32, i32, vp]),
}

_lib = None


def lib():
    """Loads the library; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(f"{LIB_PATH} is missing: run `python framework-torch-paras_amd/build.py hip`")
        l = C.CDLL(str(LIB_PATH))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name, None)
            if fn is not None:
                fn.restype, fn.argtypes = res, args
        _lib = l
    return _lib


class ParasError(RuntimeError):
    pass


def check(rc: int) -> None:
    if rc != 0:
        raise ParasError(f"status {rc}: {lib().paras_last_error().decode()}")


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


# ---------------------------------------------------------------------------
# typed helpers over CUDA tensors
# ---------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float):
    x, w = x.contiguous(), w.contiguous()
    H = x.shape[-1]
    rows = x.numel() // H if H else 0
    out = torch.empty_like(x)
    rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
    check(lib().paras_rms_norm_fwd(_ptr(x), _ptr(w), _ptr(out), _ptr(rstd), rows, H, eps, DT[x.dtype], _stream()))
    return out, rstd


def rms_norm_backward(go, x, w, rstd):
    go, x, w = go.contiguous(), x.contiguous(), w.contiguous()
    H = x.shape[-1]
    rows = x.numel() // H if H else 0
    gx = torch.empty_like(x)
    gw = torch.zeros(H, dtype=w.dtype, device=x.device)
    ws = torch.empty(max(1, lib().paras_rms_norm_bwd_workspace(rows, H)), dtype=torch.uint8, device=x.device)
    check(lib().paras_rms_norm_bwd(_ptr(go), _ptr(x), _ptr(w), _ptr(rstd), _ptr(gx), _ptr(gw), _ptr(ws), rows, H,
                                   DT[x.dtype], _stream()))
    return gx, gw


def swiglu(gate, up):
    gate, up = gate.contiguous(), up.contiguous()
    out = torch.empty_like(gate)
    check(lib().paras_swiglu_fwd(_ptr(gate), _ptr(up), _ptr(out), gate.numel(), DT[gate.dtype], _stream()))
    return out


def swiglu_backward(go, gate, up):
    go, gate, up = go.contiguous(), gate.contiguous(), up.contiguous()
    gg, gu = torch.empty_like(gate), torch.empty_like(up)
    check(lib().paras_swiglu_bwd(_ptr(go), _ptr(gate), _ptr(up), _ptr(gg), _ptr(gu), go.numel(), DT[go.dtype], _stream()))
    return gg, gu


def rotate_half(x, backward=False):
    x = x.contiguous()
    D = x.shape[-1]
    out = torch.empty_like(x)
    check(lib().paras_rotate_half(_ptr(x), _ptr(out), x.numel() // D if D else 0, D, int(backward), DT[x.dtype], _stream()))
    return out


def sdpa_args(q, k, v, out, attn=None, lse=None, mask=None, is_causal=False, scale=None) -> SdpaArgs:
    """q [B,Hq,Lq,D], k [B,Hkv,Lk,D], v [B,Hkv,Lk,Dv]; last dim contiguous."""
    import math
    a = SdpaArgs()
    B, Hq, Lq, D = q.shape
    _, Hkv, Lk, _ = k.shape
    Dv = v.shape[-1]
    assert q.stride(-1) == 1 and k.stride(-1) == 1 and v.stride(-1) == 1 and out.is_contiguous()
    a.q, a.k, a.v, a.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    a.attn = attn.data_ptr() if attn is not None else None
    a.lse = lse.data_ptr() if lse is not None else None
    a.mask_kind = 0
    if mask is not None:
        m = mask
        while m.dim() < 4:
            m = m.unsqueeze(0)
        m = m.expand(B, Hq, Lq, Lk)
        a.mask = m.data_ptr()
        a.mask_kind = 1 if mask.dtype == torch.bool else 2
        for i in range(4):
            a.mask_strides[i] = m.stride(i)
    a.is_causal = int(is_causal)
    a.dtype = DT[q.dtype]
    a.B, a.Hq, a.Hkv, a.Lq, a.Lk, a.D, a.Dv = B, Hq, Hkv, Lq, Lk, D, Dv
    for i in range(3):
        a.q_strides[i], a.k_strides[i], a.v_strides[i] = q.stride(i), k.stride(i), v.stride(i)
    a.scale = scale if scale is not None else 1.0 / math.sqrt(D)
    return a


def sdpa(q, k, v, mask=None, is_causal=False, scale=None, want_attn=False, want_lse=False):
    """Returns (out, attn or None, lse or None, kernel name)."""
    B, Hq, Lq, _ = q.shape
    Lk, Dv = k.shape[2], v.shape[-1]
    out = torch.empty(B, Hq, Lq, Dv, dtype=q.dtype, device=q.device)
    attn = torch.empty(B, Hq, Lq, Lk, dtype=q.dtype, device=q.device) if want_attn else None
    lse = torch.empty(B, Hq, Lq, dtype=torch.float32, device=q.device) if want_lse else None
    a = sdpa_args(q, k, v, out, attn, lse, mask, is_causal, scale)
    name = lib().paras_sdpa_kernel_name(C.byref(a)).decode()
    nws = lib().paras_sdpa_workspace(C.byref(a))
    ws = torch.empty(nws, dtype=torch.uint8, device=q.device) if nws else None
    check(lib().paras_sdpa_fwd(C.byref(a), _ptr(ws), _stream()))
    return out, attn, lse, name


def moe_route(logits, k, workspace=None):
    logits = logits.contiguous()
    T, E = logits.shape
    dev = logits.device
    topi = torch.empty(T, k, dtype=torch.int64, device=dev)
    topw = torch.empty(T, k, dtype=torch.float32, device=dev)
    order = torch.empty(T * k, dtype=torch.int64, device=dev)
    inv = torch.empty(T * k, dtype=torch.int64, device=dev)
    counts = torch.empty(E, dtype=torch.int64, device=dev)
    offsets = torch.empty(E + 1, dtype=torch.int64, device=dev)
    ws = workspace
    if ws is None:
        ws = torch.empty(max(1, lib().paras_moe_route_workspace(T, E, k)), dtype=torch.uint8, device=dev)
    check(lib().paras_moe_route(_ptr(logits), T, E, k, DT[logits.dtype], _ptr(topi), _ptr(topw), _ptr(order),
                                _ptr(inv), _ptr(counts), _ptr(offsets), _ptr(ws), _stream()))
    return topi, topw, order, inv, counts, offsets


def moe_route_noalloc(logits, k, out=None):
    """paras_moe_route_noalloc: the outputs are allocated here, before the call, by the caller."""
    logits = logits.contiguous()
    T, E = logits.shape
    dev = logits.device
    if out is None:
        out = (torch.empty(T, k, dtype=torch.int64, device=dev), torch.empty(T, k, dtype=torch.float32, device=dev),
               torch.empty(T * k, dtype=torch.int64, device=dev), torch.empty(T * k, dtype=torch.int64, device=dev),
               torch.empty(E, dtype=torch.int64, device=dev), torch.empty(E + 1, dtype=torch.int64, device=dev))
    topi, topw, order, inv, counts, offsets = out
    check(lib().paras_moe_route_noalloc(_ptr(logits), T, E, k, DT[logits.dtype], _ptr(topi), _ptr(topw), _ptr(order),
                                        _ptr(inv), _ptr(counts), _ptr(offsets), _stream()))
    return out


def moe_ffn(x, w_gate, w_up, w_down, topw, order, inv_order, offsets, k, workspace=None):
    T, H = x.shape
    E, I, _ = w_gate.shape
    out = torch.empty(T, H, dtype=x.dtype, device=x.device)
    if workspace is None:
        n = lib().paras_moe_ffn_workspace(T, k, H, I, DT[x.dtype])
        workspace = torch.empty(max(1, n), dtype=torch.uint8, device=x.device)
    check(lib().paras_moe_ffn(_ptr(x), _ptr(w_gate), _ptr(w_up), _ptr(w_down), _ptr(topw), _ptr(order),
                              _ptr(inv_order), _ptr(offsets), _ptr(out), _ptr(workspace), T, E, k, H, I,
                              DT[x.dtype], _stream()))
    return out


def gemm_nt(a, b, addend=None, alpha=1.0, beta=1.0, workspace=False):
    """C = alpha * a @ b^T (+ beta * addend); a [.., M, K], b [.., N, K] (2-D or batched 3-D,
    last dim contiguous); addend [N] (bias), [M, N] or [B, M, N].  workspace=True hands the
    library the workspace it asks for (paras_gemm_nt_ws)."""
    batched = a.dim() == 3
    B = a.shape[0] if batched else 1
    M, K = a.shape[-2:]
    N = b.shape[-2]
    c = torch.empty((B, M, N) if batched else (M, N), dtype=a.dtype, device=a.device)
    sa = a.stride(0) if batched else 0
    sb = b.stride(0) if (batched and b.dim() == 3) else 0
    ld_add = sadd = 0
    if addend is not None:
        if addend.dim() >= 2:
            ld_add = addend.stride(-2)
        if addend.dim() == 3:
            sadd = addend.stride(0)
    if workspace:
        nbytes = lib().paras_gemm_nt_workspace(M, N, K, B, DT[a.dtype])
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=a.device)
        check(lib().paras_gemm_nt_ws(_ptr(a), _ptr(b), _ptr(addend) if addend is not None else None, _ptr(c), M, N, K,
                                     a.stride(-2), b.stride(-2), N, ld_add, B, sa, sb, M * N, sadd, alpha, beta,
                                     DT[a.dtype], _ptr(ws), nbytes, _stream()))
        return c
    check(lib().paras_gemm_nt(_ptr(a), _ptr(b), _ptr(addend) if addend is not None else None, _ptr(c), M, N, K,
                              a.stride(-2), b.stride(-2), N, ld_add, B, sa, sb, M * N, sadd, alpha, beta,
                              DT[a.dtype], _stream()))
    return c


def softmax_rows(x, out_dtype=None):
    out_dtype = out_dtype or x.dtype
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    n = x.shape[-1] if x.dim() else 1
    rows = x.numel() // n if n else 0
    check(lib().paras_softmax_rows(_ptr(x), _ptr(out), rows, n, DT[x.dtype], DT[out_dtype], _stream()))
    return out


def topk_rows(x, k, largest=True):
    n = x.shape[-1]
    rows = x.numel() // n if n else 0
    values = torch.empty(*x.shape[:-1], k, dtype=x.dtype, device=x.device)
    indices = torch.empty(*x.shape[:-1], k, dtype=torch.int64, device=x.device)
    check(lib().paras_topk_rows(_ptr(x), _ptr(values), _ptr(indices), rows, n, k, 1 if largest else 0, DT[x.dtype], _stream()))
    return values, indices
