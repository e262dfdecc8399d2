"""Without a GPU: the package imports, registers the `paras` device and its op
schemas, reports no device, and refuses to run instead of falling back."""
import pytest
import torch


def test_import_registers_device_and_schemas():
    import torch_paras
    assert torch_paras.backend_name() == "paras-hip"
    assert torch._C._get_privateuse1_backend_name() == "paras"
    assert hasattr(torch, "paras") and callable(torch.paras.is_available)
    for name in ("rms_norm", "rms_norm_backward", "swiglu", "swiglu_backward", "rotate_half", "rotate_half_backward",
                 "moe_route", "moe_ffn"):
        assert hasattr(torch.ops.paras, name)
    s = str(torch.ops.paras.rms_norm.default._schema)
    assert s == "paras::rms_norm(Tensor input, Tensor weight, float eps) -> (Tensor, Tensor)"      # fused_ops.cpp:308
    assert str(torch.ops.torch_paras.swiglu.default._schema) == "torch_paras::swiglu(Tensor x, Tensor gate) -> Tensor"
    for op in ("aten::_scaled_dot_product_attention_math", "aten::rms_norm", "aten::_copy_from", "aten::empty.memory_format"):
        assert torch._C._dispatch_has_kernel_for_dispatch_key(op, "PrivateUse1"), op
    for fn in ("device_count", "is_available", "synchronize", "manual_seed", "manual_seed_all", "empty_cache", "device_name",
               "backend_name", "is_gpu_device", "memory_allocated", "memory_cached", "get_amp_supported_dtype"):
        assert callable(getattr(torch_paras, fn))
    assert {"rms_norm", "swiglu", "rotate_half"} <= set(torch_paras.nn.__all__)


def test_cpu_kernel_of_torch_paras_swiglu():
    import torch_paras  # noqa: F401
    x, g = torch.randn(4, 32), torch.randn(4, 32)
    assert torch.equal(torch.ops.torch_paras.swiglu(x, g), x * torch.nn.functional.silu(g))


def test_no_device_means_error_not_fallback():
    import torch_paras
    if torch_paras.device_count() > 0:
        pytest.skip("a GPU is visible: covered by the gpu tests")
    assert not torch_paras.is_available() and not torch.paras.is_available()
    with pytest.raises(RuntimeError, match="invalid device index"):
        torch.randn(4).to("paras")
    with pytest.raises(RuntimeError):
        torch.empty(4, device="paras:0")


def test_bench_refuses_more_than_one_gpu():
    """One GPU per box: asking bench.py for more must end with a message, not a rendezvous."""
    import subprocess
    import sys
    from pathlib import Path
    root = Path(__file__).resolve().parents[1]
    r = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


def test_reference_device_numbering_is_an_opt_in():
    """PARAS_DEVICE_BASE=1: `paras:0` is the reference's host-engine slot (absent from this build, so
    it raises), GPUs count from 1 (csrc/compat/paras_compat.cpp:87-97).  Runs in a child process:
    the variable is read when the extension loads."""
    import os
    import subprocess
    import sys
    from pathlib import Path
    root = Path(__file__).resolve().parents[1]
    code = (
        "import sys; sys.path.insert(0, %r)\n"
        "import torch, torch_paras\n"
        "n = torch_paras.device_count()\n"
        "assert n >= 1 and torch_paras.current_device() == 1 and torch_paras.is_gpu_device(0) is False\n"
        "assert torch_paras.is_available() == (n > 1)\n"
        "try:\n"
        "    torch.randn(4).to('paras:0')\n"
        "    raise SystemExit('paras:0 did not raise')\n"
        "except RuntimeError as e:\n"
        "    assert 'no host' in str(e), str(e)\n"
        "if n > 1:\n"
        "    x = torch.randn(8, 64)\n"
        "    d = x.to('paras:1')\n"
        "    assert d.device == torch.device('paras', 1) and torch.equal(d.cpu(), x)\n"
        "    out, rstd = torch.ops.paras.rms_norm(d.bfloat16(), torch.ones(64).bfloat16().to('paras:1'), 1e-6)\n"
        "    ref = x.bfloat16().float() * torch.rsqrt(x.bfloat16().float().pow(2).mean(-1, keepdim=True) + 1e-6)\n"
        "    assert (out.cpu().float() - ref).abs().max() < 2e-2 and out.device.index == 1\n"
        "    assert torch_paras.device_name(1) and torch_paras.memory_allocated(1) > 0\n"
        "    torch_paras.synchronize(1); torch_paras.synchronize()\n"
        "    try:\n"
        "        torch.randn(4).to('paras:%%d' %% n)\n"
        "        raise SystemExit('an index past the last GPU did not raise')\n"
        "    except RuntimeError:\n"
        "        pass\n"
        "print('ok')\n" % str(root / "framework-torch-paras_amd"))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300,
                       env={**os.environ, "PARAS_DEVICE_BASE": "1"})
    assert r.returncode == 0 and "ok" in r.stdout, r.stdout + r.stderr
