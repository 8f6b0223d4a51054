"""Build recipe for the gfx950 kernel library (``libareal_hip.so``).

The library is built in-tree with ``hipcc`` so that the shared object sits next to its
sources.  ``python -m areal_amd.build`` rebuilds it.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent / "csrc"
LIB_PATH = Path(__file__).resolve().parent / "libareal_hip.so"

# Packed fp32 VALU ops are switched off for every kernel: their results must not depend on
# whether the compiler paired two scalar float operations.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

# Elementwise kernels whose boolean outputs are compared bit-for-bit with a CPU evaluation of
# the same formulas are compiled without floating-point contraction, so a*b+c rounds twice as
# it does in the reference's separate tensor ops.
NO_CONTRACT = {"ppo_loss.hip", "gae_norm.hip", "aux_loss.hip"}


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; a ROCm toolchain is required to build areal_amd")


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _compile_one(src: Path, obj: Path) -> None:
    flags = list(HIPCC_FLAGS)
    if src.name in NO_CONTRACT:
        flags.append("-ffp-contract=off")
    cmd = [_hipcc(), *flags, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{proc.stderr}")


def build_all(verbose: bool = True) -> Path:
    """Compile every ``csrc/*.hip`` for gfx950 and link ``libareal_hip.so``."""
    build_dir = CSRC / "build"
    build_dir.mkdir(exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no .hip sources under {CSRC}")
    objs = [build_dir / (s.stem + ".o") for s in srcs]
    if verbose:
        print(f"[areal_amd.build] compiling {len(srcs)} HIP sources for gfx950", flush=True)
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        list(pool.map(_compile_one, srcs, objs))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[areal_amd.build] wrote {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build_all()
    sys.exit(0)
