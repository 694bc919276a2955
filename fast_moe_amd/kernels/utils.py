"""Kernel selector and small helpers of the operator API.

Mirrors /root/reference/kernels/utils.py:13-33.  ``KernelType`` keeps the
reference's members so that existing call sites type-check, and gains ``HIP``:
the hand-written gfx950 back-end, which is the only back-end this package ships.
``TRITON`` (the reference's GPU back-end) is served by the same HIP kernels;
``PYTORCH`` and ``TRITON_CC`` raise, because no PyTorch or CPU fallback exists
in this package.
"""
from __future__ import annotations

from enum import Enum, unique

import torch


@unique
class KernelType(Enum):
    TRITON = "TRITON"
    PYTORCH = "PYTORCH"
    TRITON_CC = "TRITON_CC"
    HIP = "HIP"


def _probe_gpu_unavailable():
    """(skip?, reason) in the form ``unittest.skipIf(*gpu_unavailable)`` takes, as the reference's
    tests use it (kernels/utils.py:20-25; there: no CUDA device, or a ROCm build).  Here a test can
    run when a ROCm device is visible and the HIP library has been built."""
    import os

    from .hip._lib import LIB_PATH
    if not torch.cuda.is_available() or torch.cuda.device_count() == 0:
        return True, "no GPU is visible"
    if not torch.version.hip:
        return True, "fast_moe_amd runs on ROCm devices (gfx950) only"
    if not os.path.exists(LIB_PATH):
        return True, f"{LIB_PATH} has not been built"
    return False, "a ROCm GPU and libfastmoe_hip.so are present"


gpu_unavailable = _probe_gpu_unavailable()


def require_hip_kernel(kernel: "KernelType", op: str) -> None:
    """Every operator funnels its ``kernel`` argument through this check."""
    if kernel in (KernelType.HIP, KernelType.TRITON):
        return
    raise NotImplementedError(
        f"{op}: kernel={kernel} is not available; fast_moe_amd ships only the MI355X HIP "
        f"back-end (KernelType.HIP, also selected by KernelType.TRITON) and has no PyTorch/CPU path")


def to_fp32_if_pytorch_kernel(x: torch.Tensor, kernel: KernelType = KernelType.PYTORCH) -> torch.Tensor:
    """kernels/utils.py:28-33 (test helper kept for signature compatibility)."""
    if kernel == KernelType.PYTORCH:
        return x.to(torch.float32)
    return x


@torch.fx.wrap
def fx_torch_zeros_like(t: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """kernels/utils.py:36-38: a leaf for fx tracing."""
    return torch.zeros_like(t, dtype=dtype)


@torch.fx.wrap
def fx_infer_max_len(lengths: torch.Tensor) -> int:
    """kernels/utils.py:41-53: the longest expert segment as a host integer (a device-to-host
    sync).  The HIP operators accept ``max_seq_len`` and ignore it, their tile scheduling reads
    the offsets on the device, so callers of this package may pass 0 and skip the sync; the
    helper stays for code that is shared with the reference's back-ends."""
    longest = int(lengths.max())
    if not torch.jit.is_scripting() and torch.compiler.is_compiling():
        torch._check_is_size(longest)      # a size in (0, 10**9) for the compiler's range analysis
        torch._check(0 < longest < 10 ** 9)
    return longest
