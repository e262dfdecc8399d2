"""Access to tests/golden/hotpath.safetensors (vectors produced by the
reference's own host engine; see tests/golden/make_golden.py)."""
from pathlib import Path

from safetensors.torch import load_file

_PATH = Path(__file__).resolve().parent / "golden" / "hotpath.safetensors"
_cache = None


def case(name: str) -> dict:
    global _cache
    if _cache is None:
        _cache = load_file(str(_PATH))
    out = {k.split("/", 1)[1]: v for k, v in _cache.items() if k.split("/", 1)[0] == name}
    assert out, f"no golden case {name}"
    return out


DTYPE_TAGS = ("f32", "bf16", "f16")
