"""bf16 operator API of the MoE forward -- the drop-in boundary.

Function names, positional order, keyword names and argument meaning are those
of /root/reference/kernels/moe.py:39-292.  Differences, all on purpose:

* ``kernel`` defaults to ``KernelType.HIP`` (the reference defaults to its
  PyTorch path, which this package does not contain); ``KernelType.TRITON`` is
  accepted and runs the same HIP kernels; any other value raises.
* every operator here has a backward (kernels/hip/autograd.py), the 3D and the two-input
  gating variants included; of the fp8 operators, silu_jagged_bmm_fp8 and silu_jagged_fp8 are
  forward only (as in the reference) and raise when an input requires grad under grad mode.
* ``max_seq_len`` is accepted and ignored: tile scheduling reads ``offsets`` on
  the device, so no host synchronisation is needed to obtain it.
* operands must be bf16 or fp32 CUDA tensors (fp32 runs true-fp32 MFMA, no tf32).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from .hip import autograd as _ag
from .hip import ops
from .hip._lib import EPI_GATED, EPI_NONE, EPI_SWIGLU
from .utils import KernelType, require_hip_kernel


@dataclass
class IndexSelectJaggedBmmOption:
    """kernels/triton/triton_moe.py:36-43: backward-tuning knobs, accepted and unused."""
    d_jagged_use_grouped_gemm: bool = True
    d_jagged_use_wrap_specialization: bool = True
    d_jagged_gemm_out_type: torch.dtype = torch.float32
    d_weight_optimization: bool = True
    d_weight_split_k_kernel: bool = True
    d_weight_split_k_kernel_tma: bool = False


@dataclass
class SiluJaggedBmmCombineOption:
    """kernels/triton/triton_moe.py:3562-3567: accepted and unused (backward only)."""
    activation_checkpointing: bool = False
    d_weight_optimization: bool = True
    d_weight_split_k_kernel: bool = True
    d_weight_split_k_kernel_tma: bool = False


def _check_gather_args(name, index, jagged, weight):
    assert index.ndim == 2 and index.shape[0] == jagged.shape[0], (
        f"{name}: index must be [L, A] with L = jagged.shape[0]")
    assert weight.ndim == 3, f"{name}: weight must be [E, K, N]"


def index_select_jagged_bmm(
    max_seq_len: int,
    offsets: torch.Tensor,
    index: torch.Tensor,
    jagged: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    kernel: KernelType = KernelType.HIP,
    triton_option: Optional[IndexSelectJaggedBmmOption] = None,
) -> torch.Tensor:
    """kernels/moe.py:39-68.  ``out[off_e:off_e+1] = jagged[index[...] // A] @ weight[e] + bias[e]``."""
    require_hip_kernel(kernel, "index_select_jagged_bmm")
    _check_gather_args("index_select_jagged_bmm", index, jagged, weight)
    if _ag.needs_grad(jagged, weight, bias):
        return _ag.IndexSelectJaggedBmm.apply(offsets, index, jagged, weight, bias, None, None)
    return ops.grouped_gemm(offsets, jagged, weight, total_rows=index.numel(), row_index=index,
                            index_div=index.shape[-1], bias=bias, epilogue=EPI_NONE)


def mul_merge_k_add(
    index: torch.Tensor,
    reverse_index: torch.Tensor,
    value: torch.Tensor,
    stable_sorting: bool = False,
    weight: Optional[torch.Tensor] = None,
    weight_index: Optional[torch.Tensor] = None,
    kernel: KernelType = KernelType.HIP,
    triton_cc_version: str = "",
) -> torch.Tensor:
    """kernels/moe.py:71-115.  ``out[n] = sum of value[r] * weight_flat[weight_index[r]]`` over the
    K rows r = reverse_index[n, :], added in ascending r."""
    require_hip_kernel(kernel, "mul_merge_k_add")
    N = index.shape[0]
    L, K = reverse_index.shape
    assert index.ndim == 1 and reverse_index.ndim == 2
    assert N == L * K and N == value.shape[0]
    if weight is not None:
        assert weight_index is not None
        assert weight.numel() == weight_index.numel() == value.shape[0], (
            f"{weight.shape=}, {weight_index.shape=}, {value.shape=}")
    if _ag.needs_grad(value, weight):
        return _ag.MulMergeKAdd.apply(index, reverse_index, value, weight, weight_index)
    return ops.combine(value, reverse_index, weight, weight_index)


def index_select_jagged_bmm_3D(
    max_seq_len: int,
    offsets: torch.Tensor,
    index: torch.Tensor,
    jagged: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor,
    kernel: KernelType = KernelType.HIP,
) -> torch.Tensor:
    """kernels/moe.py:118-153.  jagged [L, E, D_in]: expert e reads slice ``[:, e, :]``."""
    require_hip_kernel(kernel, "index_select_jagged_bmm_3D")
    assert index.ndim == 2 and index.shape[0] == jagged.shape[0]
    assert jagged.ndim == 3 and jagged.shape[1] == weight.shape[0]
    if _ag.needs_grad(jagged, weight, bias):
        return _ag.IndexSelectJaggedBmm3D.apply(offsets, index, jagged, weight, bias)
    jagged = ops._rows_contiguous(jagged)
    return ops.grouped_gemm(offsets, jagged, weight, total_rows=index.numel(), row_index=index,
                            index_div=index.shape[-1], bias=bias, epilogue=EPI_NONE,
                            a_expert_stride=jagged.stride(1))


def index_select_jagged_bmm_swiglu(
    max_seq_len: int,
    offsets: torch.Tensor,
    index: torch.Tensor,
    jagged: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    weight_p: torch.Tensor,
    bias_p: Optional[torch.Tensor],
    kernel: KernelType = KernelType.HIP,
) -> torch.Tensor:
    """kernels/moe.py:156-189.  ``silu(x W + b) * (x Wp + bp)`` in one kernel."""
    require_hip_kernel(kernel, "index_select_jagged_bmm_swiglu")
    _check_gather_args("index_select_jagged_bmm_swiglu", index, jagged, weight)
    assert weight.shape == weight_p.shape
    if weight_p.stride() != weight.stride():
        weight_p = weight_p.contiguous()
        weight = weight.contiguous()
    if _ag.needs_grad(jagged, weight, bias, weight_p, bias_p):
        return _ag.IndexSelectJaggedBmm.apply(offsets, index, jagged, weight, bias, weight_p, bias_p)
    return ops.grouped_gemm(offsets, jagged, weight, total_rows=index.numel(), row_index=index,
                            index_div=index.shape[-1], bias=bias, b2=weight_p, bias2=bias_p,
                            epilogue=EPI_SWIGLU)


def index_select_jagged_gating_bmm(
    max_seq_len: int,
    offsets: torch.Tensor,
    index: torch.Tensor,
    jagged_a: torch.Tensor,
    jagged_b: torch.Tensor,
    weight_a: torch.Tensor,
    bias_a: Optional[torch.Tensor],
    weight_b: torch.Tensor,
    bias_b: Optional[torch.Tensor],
    kernel: KernelType = KernelType.HIP,
) -> torch.Tensor:
    """kernels/moe.py:192-233.  ``silu(A Wa + ba) * (B Wb + bb)``; one fused kernel when A is B,
    otherwise two GEMMs, the second of which multiplies by the SiLU of the first one's result in
    its epilogue (bf16; fp32: two GEMMs and an element-wise kernel)."""
    require_hip_kernel(kernel, "index_select_jagged_gating_bmm")
    assert (index.ndim == 2 and index.shape[0] == jagged_a.shape[0] == jagged_b.shape[0]
            and jagged_a.shape == jagged_b.shape and weight_a.shape == weight_b.shape)
    if jagged_a is jagged_b:
        return index_select_jagged_bmm_swiglu(max_seq_len, offsets, index, jagged_a, weight_a, bias_a,
                                              weight_b, bias_b, kernel)
    if _ag.needs_grad(jagged_a, jagged_b, weight_a, weight_b, bias_a, bias_b):
        return _ag.IndexSelectJaggedGatingBmm.apply(offsets, index, jagged_a, jagged_b, weight_a, weight_b,
                                                    bias_a, bias_b)
    alpha = ops.grouped_gemm(offsets, jagged_a, weight_a, total_rows=index.numel(), row_index=index,
                             index_div=index.shape[-1], bias=bias_a)
    if jagged_a.dtype == torch.bfloat16 and index.numel() > 0:
        return ops.grouped_gemm(offsets, jagged_b, weight_b, total_rows=index.numel(), row_index=index,
                                index_div=index.shape[-1], bias=bias_b, epilogue=EPI_GATED, gate=alpha)
    beta = ops.grouped_gemm(offsets, jagged_b, weight_b, total_rows=index.numel(), row_index=index,
                            index_div=index.shape[-1], bias=bias_b)
    return ops.silu_mul(alpha, beta)


def silu_jagged_bmm_combine(
    max_seq_len: int,
    offsets: torch.Tensor,
    jagged: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    index: torch.Tensor,
    reverse_index: torch.Tensor,
    gating_scores: Optional[torch.Tensor] = None,
    gates_index: Optional[torch.Tensor] = None,
    has_silu: bool = True,
    kernel: KernelType = KernelType.HIP,
    triton_option: Optional[SiluJaggedBmmCombineOption] = None,
) -> torch.Tensor:
    """kernels/moe.py:236-292.  ``silu(jagged) @ weight[e] + bias[e]`` on expert-sorted rows, then
    the weighted merge of the K rows of each token."""
    if kernel == KernelType.TRITON_CC:
        raise NotImplementedError("TRITON_CC is not supported for silu_jagged_bmm_combine")
    require_hip_kernel(kernel, "silu_jagged_bmm_combine")
    N = index.shape[0]
    L, K = reverse_index.shape
    assert index.ndim == 1 and reverse_index.ndim == 2
    assert N == L * K and N == jagged.shape[0], f"{N=}, {L=}, {K=}, {jagged.shape=}"
    if _ag.needs_grad(jagged, weight, bias, gating_scores):
        return _ag.SiluJaggedBmmCombine.apply(offsets, jagged, weight, bias, index, reverse_index,
                                              gating_scores, gates_index, has_silu)
    bmm_out = ops.grouped_gemm(offsets, jagged, weight, total_rows=N, bias=bias, epilogue=EPI_NONE,
                               a_silu=has_silu)
    return ops.combine(bmm_out, reverse_index, gating_scores, gates_index)


def fused_jagged_bmm_swiglu_combine(
    offsets: torch.Tensor,
    index: torch.Tensor,
    jagged: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    weight_p: torch.Tensor,
    bias_p: Optional[torch.Tensor],
    weight_out: torch.Tensor,
    bias_out: Optional[torch.Tensor],
    k: int,
    gates: Optional[torch.Tensor] = None,
    gates_index: Optional[torch.Tensor] = None,
    kernel: KernelType = KernelType.HIP,
) -> torch.Tensor:
    """kernels/pytorch/moe.py:306-391 (pytorch_fused_jagged_bmm_swiglu_combine): the whole expert
    block of a SwiGLU MoE, ``merge_k(gates * ((silu(x W + b) * (x Wp + bp)) W_out + b_out))`` ->
    [L, D].  Three launches (gather + SwiGLU GEMM, down GEMM, merge); differentiable through the
    two operators it is made of."""
    require_hip_kernel(kernel, "fused_jagged_bmm_swiglu_combine")
    assert index.ndim == 2 and index.shape[1] == k, f"{index.shape=}, {k=}"
    hidden = index_select_jagged_bmm_swiglu(0, offsets, index, jagged, weight, bias, weight_p, bias_p, kernel)
    token_index = torch.div(index.reshape(-1), k, rounding_mode="floor")
    reverse_index = _ag._reverse_from_index(index)
    return silu_jagged_bmm_combine(0, offsets, hidden, weight_out, bias_out, token_index, reverse_index,
                                   gates, gates_index, has_silu=False, kernel=kernel)
