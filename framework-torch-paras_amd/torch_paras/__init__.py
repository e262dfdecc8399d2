"""`paras` PyTorch device on AMD MI355X.

Importing the package registers the device with PyTorch::

    import torch, torch_paras
    x = torch.randn(16384, 4096, dtype=torch.bfloat16, device="paras")   # paras:0 = first MI355X
    y = torch_paras.nn.rms_norm(x, w)
    o = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)

Public names follow the reference package (python/torch_paras/__init__.py:46-139):
device_count, is_available, synchronize, manual_seed(_all), empty_cache,
device_name, backend_name, is_gpu_device, memory_allocated, memory_cached,
get_amp_supported_dtype, and the ``nn`` submodule.  One difference in device
numbering, on purpose: this build is HIP-only, so ``paras:i`` is HIP GPU ``i``;
there is no host-CPU engine behind ``paras:0``.  Scripts written for the
reference's numbering (``paras:0`` = host engine, GPUs from ``paras:1``) run
unchanged with ``PARAS_DEVICE_BASE=1`` in the environment before the import:
``paras:i`` is then HIP GPU ``i - 1``, ``device_count()`` counts the host slot
as the reference does, and any use of ``paras:0`` raises.  With no GPU visible
the package still imports and every op on a ``paras`` tensor raises.
"""
from __future__ import annotations

import types

import torch

from . import _C
from . import nn  # noqa: F401

__all__ = [
    "device_count", "is_available", "synchronize", "manual_seed", "manual_seed_all", "empty_cache",
    "device_name", "backend_name", "is_gpu_device", "memory_allocated", "memory_cached",
    "get_amp_supported_dtype", "current_device", "nn",
]


def device_count() -> int:
    """Number of paras device indices: the visible HIP GPUs, plus the (unusable) host
    slot ``paras:0`` under PARAS_DEVICE_BASE=1."""
    return _C.device_count()


def is_available() -> bool:
    return device_count() - _C.device_base() > 0


def backend_name() -> str:
    """Always 'paras-hip' for this build."""
    return _C.backend_name()


def device_name(device: int = 0) -> str:
    return _C.device_name(device)


def is_gpu_device(device: int) -> bool:
    return _C.is_gpu_device(device)


def current_device() -> int:
    return _C.current_device()


def synchronize(device: int | None = None) -> None:
    """Waits for the work queued on one device, or on all of them."""
    if device is None:
        _C.synchronize_all()
    else:
        _C.synchronize(device)


def manual_seed(seed: int, device: int | None = None) -> None:
    if device is None:
        _C.manual_seed_all(seed)
    else:
        _C.manual_seed(device, seed)


def manual_seed_all(seed: int) -> None:
    _C.manual_seed_all(seed)


def empty_cache() -> None:
    """Hands the blocks cached by the HBM pools back to the driver."""
    _C.empty_cache()


def memory_allocated(device: int = 0) -> int:
    return _C.allocated_bytes(device)


def memory_cached(device: int = 0) -> int:
    return _C.cached_bytes(device)


def get_amp_supported_dtype() -> list[torch.dtype]:
    return [torch.float16, torch.float32]


def _register() -> None:
    torch.utils.rename_privateuse1_backend("paras")
    mod = types.ModuleType("torch.paras")
    for name in ("device_count", "is_available", "synchronize", "manual_seed", "manual_seed_all", "empty_cache",
                 "device_name", "current_device", "get_amp_supported_dtype"):
        setattr(mod, name, globals()[name])
    mod.is_bad_fork = _C.is_bad_fork
    mod._is_in_bad_fork = _C.is_bad_fork
    torch._register_device_module("paras", mod)
    # tensor.paras() / module.paras() / tensor.is_paras
    torch.utils.generate_methods_for_privateuse1_backend(for_tensor=True, for_module=True, for_storage=False)


_register()
