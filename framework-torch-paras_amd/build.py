"""In-tree build of the native pieces.

    python framework-torch-paras_amd/build.py [hip] [torch] [oracle] [ref]

* ``hip``    libparas_hip.so: device context + HBM pool + every HIP kernel,
             compiled by hipcc for gfx950 only, exporting the C ABI declared
             in include/paras_hip.h.  No torch types inside.
* ``torch``  torch_paras/_C.so: the PyTorch side (PrivateUse1 device `paras`,
             allocator adapter, op registrations, pybind functions), compiled
             by g++ against the torch headers and linked to libparas_hip.so.
* ``oracle`` oracle/libparas_oracle.so: the CPU restatement used by tests and
             by bench.py's cpu_baseline leg.
* ``ref``    oracle/_ref/libparas_ref.so: the reference's own CPU flavor,
             built from /root/reference when that tree is present.

With no argument everything that can be built is built.  Objects are compiled
in parallel (one hipcc / g++ process per translation unit).
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import shutil
import subprocess
import sys
import sysconfig
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
OUT = PKG / "torch_paras" / "lib"
OBJ = PKG / "build"
INCLUDE = ROOT / "include"
ROCM = Path(os.environ.get("ROCM_PATH", "/opt/rocm"))
HIPCC = os.environ.get("HIPCC", str(ROCM / "bin" / "hipcc"))
ARCH = "gfx950"
JOBS = int(os.environ.get("MAX_JOBS", "8"))

HIP_FLAGS = [
    "-O3", f"--offload-arch={ARCH}", "-fPIC", "-std=c++17", "-fvisibility=hidden",
    # Packed-fp32 VALU forms are kept out of every kernel of this library.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-option-ignored",
    f"-I{INCLUDE}", f"-I{CSRC}",
]


def _run(cmd: list[str], what: str) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"{what} failed:\n{' '.join(cmd)}\n{proc.stdout}\n{err}")
    if err.strip():
        print(err, file=sys.stderr)


def _newer(src: Path, dst: Path, extra: list[Path]) -> bool:
    if not dst.exists():
        return True
    t = dst.stat().st_mtime
    return any(p.stat().st_mtime > t for p in [src, *extra])


def _compile_all(units: list[tuple[list[str], Path, Path]], headers: list[Path], force: bool) -> list[Path]:
    """units: (command prefix, source, object).  Returns the objects."""
    todo = [(c, s, o) for c, s, o in units if force or _newer(s, o, headers)]
    for _, _, o in todo:
        o.parent.mkdir(parents=True, exist_ok=True)
    with cf.ThreadPoolExecutor(max_workers=JOBS) as ex:
        futs = [ex.submit(_run, [*c, "-c", str(s), "-o", str(o)], f"compile {s.name}") for c, s, o in todo]
        for f in futs:
            f.result()
    return [o for _, _, o in units]


def build_hip(force: bool = True) -> Path:
    if shutil.which(HIPCC) is None:
        raise RuntimeError(f"hipcc not found at {HIPCC}")
    srcs = sorted((CSRC / "core").glob("*.cpp")) + sorted((CSRC / "kernels").glob("*.hip"))
    headers = list(CSRC.rglob("*.h")) + list(INCLUDE.glob("*.h"))
    units = []
    for s in srcs:
        cmd = [HIPCC, *HIP_FLAGS]
        if s.suffix == ".cpp":
            cmd += ["-x", "hip"]
        units.append((cmd, s, OBJ / "hip" / (s.stem + ".o")))
    objs = _compile_all(units, headers, force)
    OUT.mkdir(parents=True, exist_ok=True)
    lib = OUT / "libparas_hip.so"
    _run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", str(lib), *map(str, objs),
          f"-Wl,-rpath,{ROCM / 'lib'}"], "link libparas_hip.so")
    return lib


def build_torch(force: bool = True) -> Path:
    import torch  # noqa: F401  (headers and libs come from the installed wheel)
    tdir = Path(torch.__file__).resolve().parent
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    pyinc = sysconfig.get_paths()["include"]
    import pybind11
    flags = [
        "g++", "-O2", "-fPIC", "-std=c++17", "-fvisibility=hidden", "-w",
        f"-D_GLIBCXX_USE_CXX11_ABI={abi}", "-DTORCH_API_INCLUDE_EXTENSION_H", "-DTORCH_EXTENSION_NAME=_C",
        f"-I{INCLUDE}", f"-I{CSRC}", "-isystem", str(tdir / "include"),
        "-isystem", str(tdir / "include" / "torch" / "csrc" / "api" / "include"),
        "-isystem", pyinc, "-isystem", pybind11.get_include(),
    ]
    srcs = sorted((CSRC / "torch").glob("*.cpp"))
    headers = list((CSRC / "torch").glob("*.h")) + list(INCLUDE.glob("*.h"))
    units = [(flags, s, OBJ / "torch" / (s.stem + ".o")) for s in srcs]
    objs = _compile_all(units, headers, force)
    lib = PKG / "torch_paras" / "_C.so"
    _run(["g++", "-shared", "-o", str(lib), *map(str, objs), f"-L{OUT}", "-lparas_hip",
          f"-L{tdir / 'lib'}", "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10", "-lpthread",
          "-Wl,-rpath,$ORIGIN/lib", f"-Wl,-rpath,{tdir / 'lib'}"], "link _C.so")
    return lib


def build_oracle(force: bool = True) -> Path:
    src = ROOT / "oracle" / "paras_oracle.c"
    lib = ROOT / "oracle" / "libparas_oracle.so"
    if force or _newer(src, lib, []):
        _run(["gcc", "-O2", "-fPIC", "-shared", "-std=c11", "-fopenmp", "-ffp-contract=off", "-o", str(lib),
              str(src), "-lm"], "build oracle")
    return lib


def build_ref() -> Path | None:
    """The reference's CPU flavor, only where its sources are present."""
    if not Path("/root/reference/csrc").is_dir():
        return None
    _run(["make", "-f", str(ROOT / "oracle" / "Makefile.ref"), f"-j{JOBS}"], "build oracle/_ref")
    return ROOT / "oracle" / "_ref" / "libparas_ref.so"


def main(argv: list[str]) -> None:
    what = argv or ["hip", "torch", "oracle", "ref"]
    if "hip" in what:
        print("built", build_hip())
    if "torch" in what and (CSRC / "torch").exists() and list((CSRC / "torch").glob("*.cpp")):
        print("built", build_torch())
    if "oracle" in what:
        print("built", build_oracle())
    if "ref" in what:
        print("built", build_ref())


if __name__ == "__main__":
    main(sys.argv[1:])
