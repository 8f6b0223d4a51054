"""ctypes binding of ``libareal_hip.so`` (the C ABI declared in ``include/areal_hip.h``).

There is no CPU implementation behind these entry points: if the library is missing or a
tensor is not on a HIP device the call raises.
"""

from __future__ import annotations

import ctypes
import functools
import re
import shutil
import subprocess
from ctypes import c_float, c_double, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

import torch

LIB_PATH = Path(__file__).resolve().parent / "libareal_hip.so"

_STATUS = {
    0: "ok",
    -1: "bad argument",
    -2: "pointer or leading dimension not suitably aligned",
    -3: "workspace too small",
    -4: "kernel launch failed",
    -5: "unsupported shape",
}

P = c_void_p
I64 = c_int64
F = c_float
D = c_double
I = c_int
SZ = c_size_t

ABI_VERSION = 3  # AREAL_HIP_ABI_VERSION of include/areal_hip.h

# name -> (restype, argtypes).  Must list every symbol declared in include/areal_hip.h.
SIGNATURES: dict[str, tuple] = {
    "areal_gemm_nt_bf16": (I, [P, I64, P, I64, P, I64, I64, I64, I64, I, P]),
    "areal_lmhead_fwd_workspace_bytes": (SZ, [I64, I64, I64]),
    "areal_abi_version": (I, []),
    "areal_lmhead_probs_bytes": (SZ, [I64, I64]),
    "areal_lmhead_fwd": (
        I,
        [P, P, P, P, I64, I64, I64, F, F, P, P, P, P, P, P, P, P, P, SZ, P, P, P, SZ, P],
    ),
    "areal_lmhead_bwd_workspace_bytes": (SZ, [I64, I64, I64, I64]),
    "areal_lmhead_bwd": (
        I,
        [P, P, P, P, P, P, P, I64, I64, I64, F, F, P, P, P, I, I64, P, SZ, P],
    ),
    "areal_lmhead_bwd_saved_workspace_bytes": (SZ, [I64, I64, I64]),
    "areal_lmhead_bwd_saved": (
        I,
        [P, P, P, P, P, P, P, I64, I64, I64, F, F, P, SZ, P, P, P, P, I, P, P, SZ, P],
    ),
    "areal_cast_f32_to_bf16": (I, [P, P, I64, P]),
    "areal_logits_logprobs_entropy_fwd": (I, [P, I, I64, P, I64, I64, F, P, P, P, P]),
    "areal_logits_logprobs_entropy_bwd": (
        I,
        [P, I, I64, P, I64, I64, F, P, P, P, P, P, I64, P],
    ),
    "areal_actor_loss_workspace_bytes": (SZ, [I64, I64]),
    "areal_actor_loss": (
        I,
        [P, P, P, P, P, P, I64, I64, I64, P, P, P, P, P, P, P, P, P, P, P, P, P, P, SZ, P],
    ),
    "areal_actor_loss_stats_workspace_bytes": (SZ, [I64, I64]),
    "areal_actor_loss_stats": (
        I,
        [P, P, P, P, P, P, I64, I64, I64, P, P, P, P, P, P, P, P, P, P, P, P, P, P, P, P, P, P, SZ, P],
    ),
    "areal_actor_loss_static": (
        I,
        [P, P, P, P, P, P, I64, I64, I64, P, P, P, P, P, P, P, P, P, P, P, P, P, P],
    ),
    "areal_actor_loss_grad": (I, [P, P, P, P, I64, P]),
    "areal_aux_loss_workspace_bytes": (SZ, [I64, I64]),
    "areal_sapo_loss": (
        I,
        [P, P, P, P, P, I64, I64, I64, F, F, I, P, P, P, P, P, P, P, P, P, P, P, P, P, P, SZ, P],
    ),
    "areal_critic_loss": (I, [P, P, P, P, I64, F, I, P, P, P, P, P, P, SZ, P]),
    "areal_m2po_mask_workspace_bytes": (SZ, [I64]),
    "areal_m2po_mask": (I, [P, P, P, I64, F, P, P, SZ, P]),
    "areal_prox_logp_approx": (I, [P, P, P, I64, I, I, P, P]),
    "areal_distill_terms": (I, [P, P, P, P, I64, I, P, P, P, P, P, SZ, P]),
    "areal_dpo_seq_logps": (I, [P, P, P, P, I64, I64, P, P, P]),
    "areal_dpo_seq_logps_grad": (I, [P, P, P, I64, I64, P, P]),
    "areal_gae_workspace_bytes": (SZ, [I64]),
    "areal_gae_packed": (
        I,
        [P, P, P, P, P, P, I64, I64, I64, F, F, P, P, P, SZ, P],
    ),
    "areal_gae_padded_row_stats": (I, [P, P, P, P, P, I64, I64, F, F, P, P, P, P]),
    "areal_group_norm_from_row_stats": (I, [P, P, I64, I64, P, P, I64, I64, I, I, I, I, D, P, P, P]),
    "areal_gae_segment_stats_bytes": (SZ, [I64, I64]),
    "areal_gae_packed_group_stats": (I, [P, P, P, P, P, P, I64, I64, F, F, P, I64, P, P, P, SZ, P]),
    "areal_group_norm_from_segment_stats": (I, [P, P, I64, P, P, I64, I64, I, I, I, I, D, P, P, P]),
    "areal_seqlens_from_mask": (I, [P, I64, I64, P, P, P, P]),
    "areal_pack_padded": (I, [P, P, P, I64, I64, I64, I64, P]),
    "areal_pack_padded_multi": (I, [P, P, P, I, P, I64, I64, I64, P]),
    "areal_unpack_to_padded": (I, [P, P, P, P, I64, I64, I64, P, I, P]),
    "areal_realign_packed": (I, [P, P, P, I64, P, I64, I64, P, I, I, I64, P]),
    "areal_masked_stats_workspace_bytes": (SZ, [I]),
    "areal_masked_stats": (I, [P, P, I, I64, P, P, SZ, P]),
    "areal_turn_gae_workspace_bytes": (SZ, [I64, I64]),
    "areal_turn_gae": (I, [P, P, P, P, P, P, I64, I64, F, F, P, P, P, P, SZ, P]),
    "areal_gae_lambda_context": (I, [P, P, I64, I64, P, P, P, P]),
    "areal_group_norm_workspace_bytes": (SZ, [I64, I64]),
    "areal_group_norm": (
        I,
        [P, P, I64, P, P, I64, I64, I, I, I, I, I, D, P, P, SZ, P],
    ),
    "areal_masked_norm_workspace_bytes": (SZ, [I64]),
    "areal_masked_norm": (I, [P, P, I64, I, D, P, P, SZ, P]),
    "areal_masked_norm_rows": (I, [P, P, I64, I64, I, D, P, P]),
    "areal_advantage_prep": (I, [P, P, P, P, P, I64, I64, I, I, I, I, I, F, P, P, P, P, P, P, P, P, P]),
}


class LossConfig(ctypes.Structure):
    """Mirror of ``areal_loss_config`` in include/areal_hip.h (a host-side struct)."""

    _fields_ = [
        ("loss_kind", c_int),
        ("clip_lo", c_float),
        ("clip_hi", c_float),
        ("has_c_clip", c_int),
        ("c_clip", c_float),
        ("seq_is", c_int),
        ("rs_enabled", c_int),
        ("rs_seq_level", c_int),
        ("rs_clamp", c_int),
        ("rs_metric", c_int),
        ("rs_agg", c_int),
        ("rs_upper", c_float),
        ("rs_has_lower", c_int),
        ("rs_lower", c_float),
    ]

_lib = None


ERR_UNSUPPORTED = -5  # AREAL_ERR_UNSUPPORTED


class ArealHipError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load the kernel library, raising if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ArealHipError(
            f"{LIB_PATH} is missing: build it with `python -m areal_amd.build` "
            "(areal_amd has no CPU fallback)"
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    # the argument lists above are those of one version of the interface (include/areal_hip.h)
    built = lib.areal_abi_version()
    if built != ABI_VERSION:
        raise ArealHipError(
            f"{LIB_PATH} was built with interface version {built}, this package binds version "
            f"{ABI_VERSION}: rebuild it with `python -m areal_amd.build`"
        )
    _lib = lib
    return lib


@functools.lru_cache(maxsize=1)
def kernel_names() -> frozenset[str]:
    """Names of the GPU kernels the built library launches, as a profiler prints them (demangled,
    without the anonymous-namespace qualifier and the argument list), read from the launch stubs
    in the shared object. Used to keep the kernel names quoted in benchmark output honest."""
    symbols = sorted({m.decode() for m in re.findall(rb"_Z[A-Za-z0-9_]{4,600}", LIB_PATH.read_bytes())})
    tool = shutil.which("c++filt") or shutil.which("llvm-cxxfilt") or "/opt/rocm/llvm/bin/llvm-cxxfilt"
    out = subprocess.run([tool], input="\n".join(symbols), capture_output=True, text=True, check=True).stdout
    names = set()
    for line in out.splitlines():
        line = line.replace("(anonymous namespace)::", "")
        if line.startswith("void "):
            line = line[5:]
        depth, cut = 0, len(line)
        for i, ch in enumerate(line):  # cut at the argument list: the first '(' outside <...>
            if ch == "<":
                depth += 1
            elif ch == ">":
                depth -= 1
            elif ch == "(" and depth == 0:
                cut = i
                break
        names.add(line[:cut].strip())
    return frozenset(names)


def has_kernel(name: str) -> bool:
    """True for a kernel of the library; template arguments may be left out (``loss_token_kernel``
    matches ``loss_token_kernel<false>``)."""
    names = kernel_names()
    for cand in (name, "__device_stub__" + name):
        if cand in names or any(n.startswith(cand + "<") for n in names):
            return True
    return False


def check(status: int, what: str) -> None:
    if status != 0:
        raise ArealHipError(f"{what} failed: {_STATUS.get(status, status)} (code {status})")


def workspace(nbytes: int, device: torch.device) -> torch.Tensor:
    """Scratch buffer owned by the caller (PyTorch's caching allocator)."""
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


def ptr(t: torch.Tensor | None) -> c_void_p:
    """Device pointer of a tensor (None -> NULL)."""
    if t is None:
        return c_void_p(0)
    return c_void_p(t.data_ptr())


def stream_ptr(device: torch.device) -> c_void_p:
    return c_void_p(torch.cuda.current_stream(device).cuda_stream)


def require_gpu(*tensors: torch.Tensor | None) -> torch.device:
    """All given tensors must live on one HIP device; returns it."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise ArealHipError(
                "areal_amd kernels run on an MI355X only; got a tensor on "
                f"{t.device} (there is no CPU fallback)"
            )
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise ArealHipError(f"tensors on different devices: {dev} and {t.device}")
    if dev is None:
        raise ArealHipError("no tensor given")
    return dev
