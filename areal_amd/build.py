"""Build recipe for the gfx950 kernel library (``libareal_hip.so``).

The library is built in-tree with ``hipcc`` so that the shared object sits next to its
sources.  ``python -m areal_amd.build`` rebuilds it.
"""

from __future__ import annotations

import importlib.util
import os
import re
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


def generate_mainloop() -> Path:
    """Write ``csrc/mainloop16.inc``, the hand-scheduled k-loop that ``lmhead.hip`` includes."""
    spec = importlib.util.spec_from_file_location("gen_mainloop16", CSRC / "gen_mainloop16.py")
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    path = CSRC / "mainloop16.inc"
    text = gen.emit()
    if not path.exists() or path.read_text() != text:
        path.write_text(text)
    return path


def check_accumulator_registers(asm_text: str) -> int:
    """Verify what the hand-scheduled kernels rely on, on the compiler's own output.

    ``gemm16_sweep`` keeps its 256 accumulators in ``a[0:255]`` between assembly blocks without
    the compiler knowing (the main loop only lists them as clobbered, and the epilogues fetch
    them with ``v_accvgpr_read`` blocks).  That is sound as long as no instruction the compiler
    emits itself in those kernels touches an accumulator register, e.g. to park a spilled VGPR
    there.  Returns the number of kernels checked; raises if one fails.
    """
    checked = 0
    for m in re.finditer(r"^(\S*gemm16_sweep\S*):[^\n]*\n(.*?)^\.Lfunc_end", asm_text, re.S | re.M):
        name, body = m.group(1), m.group(2)
        in_block = False
        for line in body.split("\n"):
            if "#ASMSTART" in line:
                in_block = True
            elif "#ASMEND" in line:
                in_block = False
            elif not in_block:
                code = line.split(";")[0]
                if re.search(r"\ba(\d+|\[\d+:\d+\])(?![\w.])", code):
                    raise RuntimeError(f"compiler-generated use of an accumulator register in {name}:\n{line}")
        checked += 1
    if checked == 0:
        raise RuntimeError("no gemm16_sweep kernel found in the device assembly of lmhead.hip")
    return checked


def _check_lmhead(build_dir: Path) -> None:
    asm = build_dir / "lmhead.gfx950.s"
    cmd = [_hipcc(), *HIPCC_FLAGS, "--cuda-device-only", "-S", str(CSRC / "lmhead.hip"), "-o", str(asm)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc -S failed for lmhead.hip:\n{proc.stderr}")
    check_accumulator_registers(asm.read_text())


def _up_to_date(src: Path, obj: Path) -> bool:
    if not obj.exists():
        return False
    deps = [src, CSRC / "common.hpp", Path(__file__)]
    if src.name == "lmhead.hip":
        deps.append(CSRC / "mainloop16.inc")
    return all(obj.stat().st_mtime > d.stat().st_mtime for d in deps)


def build_all(verbose: bool = True, incremental: bool = False) -> Path:
    """Compile every ``csrc/*.hip`` for gfx950 and link ``libareal_hip.so``.  ``incremental``
    (``python -m areal_amd.build --incremental``, for work on one kernel file) leaves alone the
    objects that are newer than their source, the shared header and this recipe."""
    build_dir = CSRC / "build"
    build_dir.mkdir(exist_ok=True)
    generate_mainloop()
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no .hip sources under {CSRC}")
    objs = [build_dir / (s.stem + ".o") for s in srcs]
    todo = [(s, o) for s, o in zip(srcs, objs) if not (incremental and _up_to_date(s, o))]
    if verbose:
        print(f"[areal_amd.build] compiling {len(todo)} of {len(srcs)} HIP sources for gfx950", flush=True)
    with ThreadPoolExecutor(max_workers=min(8, len(srcs) + 1)) as pool:
        check = None
        if any(s.name == "lmhead.hip" for s, _ in todo):
            check = pool.submit(_check_lmhead, build_dir)
        list(pool.map(lambda so: _compile_one(*so), todo))
        if check is not None:
            check.result()
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
    build_all(incremental="--incremental" in sys.argv[1:])
    sys.exit(0)
