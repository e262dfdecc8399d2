"""The C-ABI library loads without a GPU and exports every function that
include/paras_hip.h declares (no compute calls here)."""
import ctypes
import re
from pathlib import Path

import capi

ROOT = Path(__file__).resolve().parent.parent


def declared_functions():
    text = (ROOT / "include" / "paras_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"PARAS_API\s+[\w\s\*]+?\b(paras_\w+)\s*\(", text)))


def test_header_declares_the_hot_path():
    names = declared_functions()
    for must in ("paras_rms_norm_fwd", "paras_swiglu_fwd", "paras_sdpa_fwd", "paras_moe_route", "paras_moe_ffn",
                 "paras_alloc", "paras_free", "paras_stream"):
        assert must in names


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(str(capi.LIB_PATH))
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, f"declared in paras_hip.h but not exported: {missing}"


def test_binding_table_matches_header():
    assert sorted(capi.SIGNATURES) == declared_functions()


def test_no_device_is_an_error_not_a_fallback():
    """Without a GPU the context is empty and compute entry points refuse to run."""
    import torch
    lib = capi.lib()
    assert lib.paras_abi_version() == 1
    if lib.paras_device_count() > 0:
        return  # on a GPU box the parity tests cover the calls
    x = torch.zeros(4, 8)
    rc = lib.paras_rms_norm_fwd(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), 4, 8, 1e-6, 0, None)
    assert rc == -4 and b"no HIP device" in lib.paras_last_error()
    p = ctypes.c_void_p()
    assert lib.paras_alloc(0, 1024, ctypes.byref(p)) != 0


def test_pool_size_classes():
    """Power-of-two bins of at least 256 bytes (reference pool: csrc/core/allocator.cpp:53-59)."""
    lib = capi.lib()
    for n, want in ((0, 256), (1, 256), (256, 256), (257, 512), (1000, 1024), (4096, 4096), (4097, 8192),
                    (1 << 30, 1 << 30)):
        assert lib.paras_round_size(n) == want
    big = (1 << 30) + 1
    got = lib.paras_round_size(big)
    assert got >= big and got % (256 << 20) == 0 and got - big < (256 << 20)
