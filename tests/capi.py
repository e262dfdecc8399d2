"""The ctypes binding of libparas_hip.so lives beside the package (paras_capi.py: bench.py and the
smoke test use it too); the tests keep importing it under this name."""
import sys
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent.parent / "framework-torch-paras_amd"))
import paras_capi as _impl  # noqa: E402

sys.modules[__name__] = _impl
