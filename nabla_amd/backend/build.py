"""Build libnbk.so (the gfx950 kernel library) in-tree with hipcc.

Every ``*.hip`` file under ``nabla_amd/csrc`` is compiled to an object file for
``gfx950`` and linked into ``nabla_amd/csrc/libnbk.so``.  hipcc cross-compiles,
so this runs on machines without a GPU.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parents[2]
CSRC = ROOT / "nabla_amd" / "csrc"
INCLUDE = ROOT / "include"
LIB = CSRC / "libnbk.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    # keep packed-fp32 VALU forms out of the device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _compile(src: Path, force: bool) -> Path:
    obj = src.with_suffix(".o")
    deps = [src, *CSRC.glob("*.h"), *INCLUDE.glob("*.h")]
    if not force and obj.exists() and all(obj.stat().st_mtime > d.stat().st_mtime for d in deps):
        return obj
    cmd = [HIPCC, *FLAGS, *os.environ.get("NBK_EXTRA_HIPCC_FLAGS", "").split(), "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{res.stderr[-4000:]}")
    return obj


def build(force: bool = True, jobs: int = 8, verbose: bool = False) -> Path:
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB),
           *[str(o) for o in objs], "-ldl"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link of {LIB.name} failed:\n{res.stderr[-4000:]}")
    if verbose:
        print(f"built {LIB} from {len(objs)} objects")
    return LIB


def build_examples(force: bool = True) -> list[Path]:
    """Compile the example custom-kernel libraries under tests/custom_kernels:
    every ``<name>.hip`` becomes ``lib<name>.so`` next to it."""
    out = []
    for src in sorted((ROOT / "tests" / "custom_kernels").glob("*.hip")):
        lib = src.parent / f"lib{src.stem}.so"
        if not force and lib.exists() and lib.stat().st_mtime > src.stat().st_mtime:
            out.append(lib)
            continue
        cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               f"-I{INCLUDE}", str(src), "-o", str(lib)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src.name}:\n{res.stderr[-4000:]}")
        out.append(lib)
    return out


if __name__ == "__main__":
    build(force="--force" in sys.argv, verbose=True)
    build_examples(force=True)
