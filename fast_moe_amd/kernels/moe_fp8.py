"""FP8 (OCP e4m3fn, row-wise power-of-two scales) operator API.

Names, argument order and meaning follow /root/reference/kernels/moe_fp8.py:31-248.
``kernel`` defaults to ``KernelType.HIP``; ``TRITON`` selects the same kernels.
Where the reference's two back-ends disagree on a weight layout
(kernels/triton/triton_moe_fp8.py:1393 reads [E, D_out, D_in] while the PyTorch
branch of the same operator reads [E, D_in, D_out]) the layout of the PyTorch
branch -- the one every bf16 operator uses -- is taken: weights are [E, D_in, D_out]
tensors of any strides, except ``silu_jagged_bmm_fp8`` which keeps the
[E, D_out, D_in] layout of its only runnable reference implementation.
"""
from __future__ import annotations

import weakref
from typing import Optional, Tuple

import torch

from .hip import autograd as _ag
from .hip import ops
from .hip._lib import EPI_NONE
from .utils import KernelType, require_hip_kernel


def rowwise_quant_fp8(a: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """kernels/pytorch/quant_fp8.py:27-34: ``(a_fp8, a_scale)`` with the MULTIPLIER scale."""
    return ops.quant_rows_fp8(a)


def transpose_rowwise_quant_fp8(a: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """kernels/pytorch/quant_fp8.py:37-40: quantise ``a.transpose(-2, -1)`` row-wise (no copy of a)."""
    return ops.quant_rows_fp8(a.transpose(-2, -1))


def quantize_expert_weights(weight: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Weight [E, K, N] (any strides) -> (fp8 [E, K, N] view of [E, N, K] storage, scale [E, N]):
    one scale per (expert, output row), K-contiguous bytes ready for the fp8 GEMM.  This is the
    quantisation kernels/pytorch/moe_fp8.py:111 redoes on every call; do it once per weight update."""
    q, s = ops.quant_rows_fp8(weight.permute(0, 2, 1))     # [E, N, K] contiguous
    return q.permute(0, 2, 1), s


class _WeightQuantCache:
    """(fp8 bytes, scales) of expert weights, kept until the weight changes.  OPT-IN: the
    operators below quantise their weight on every call, as the reference does
    (kernels/pytorch/moe_fp8.py:111, kernels/triton/triton_moe_fp8.py:1157, 1423: 3 bytes of
    HBM traffic per weight element per forward); a caller that wants to pay that once per weight
    update passes ``fp8_weight=cached_quantize_expert_weights(w)`` (or its own pair).

    An entry is keyed by the tensor that owns the storage (the parameter behind a
    ``permute``/``to`` view, held weakly) and by the view's geometry; it is dropped when the
    owner's in-place version counter moves (an optimizer step, ``copy_``, ``load_state_dict``)
    or the owner dies; dead owners are purged on every insert.  Out-of-place replacement
    (``layer.w = new``) makes a new owner and therefore a new entry.

    What the version counter does NOT see: writes through ``param.data`` (``p.data.mul_()``,
    hand-written optimizers, EMA updates, flat-parameter swaps that keep the pointer).  After
    such a write call ``invalidate(weight)`` (or ``clear()``), or do not use the cache.
    """

    def __init__(self, max_entries: int = 32) -> None:
        self._entries: "dict[int, tuple]" = {}
        self._max = max_entries
        self.hits = 0
        self.misses = 0

    @staticmethod
    def _owner(weight: torch.Tensor) -> torch.Tensor:
        return weight._base if weight._base is not None else weight

    def get(self, weight: torch.Tensor, quantize) -> Tuple[torch.Tensor, torch.Tensor]:
        owner = self._owner(weight)
        geom = (weight.data_ptr(), tuple(weight.shape), tuple(weight.stride()), weight.dtype, str(weight.device))
        key = id(owner)
        hit = self._entries.get(key)
        if hit is not None:
            ref, version, cached_geom, value = hit
            if ref() is owner and version == owner._version and cached_geom == geom:
                self.hits += 1
                return value
        self.misses += 1
        value = quantize(weight)
        for k in [k for k, (r, *_rest) in self._entries.items() if r() is None]:
            self._entries.pop(k, None)
        self._entries.pop(key, None)
        while len(self._entries) >= self._max:
            self._entries.pop(next(iter(self._entries)))
        self._entries[key] = (weakref.ref(owner), owner._version, geom, value)
        return value

    def invalidate(self, weight: torch.Tensor) -> None:
        """Drop the entry of the tensor that owns ``weight``'s storage (after a write the
        version counter cannot see)."""
        self._entries.pop(id(self._owner(weight)), None)

    def clear(self) -> None:
        self._entries.clear()


weight_quant_cache = _WeightQuantCache()


def cached_quantize_expert_weights(weight: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``quantize_expert_weights`` through ``weight_quant_cache`` (see its caveat on ``.data``
    writes); the result is what the operators take as ``fp8_weight``."""
    return weight_quant_cache.get(weight, quantize_expert_weights)


def _weight_pair(weight: torch.Tensor, fp8_weight) -> Tuple[torch.Tensor, torch.Tensor]:
    """The (e4m3 [E, K, N], scale [E, N]) pair of ``weight``: the caller's, checked for shape, or a
    fresh quantisation.  (A caller's own pair may carry any positive scales: the GEMM takes the
    scales for powers of two only when they are tensors this package's quantiser returned,
    ``ops.scales_are_pow2``.)"""
    if fp8_weight is None:
        return quantize_expert_weights(weight)
    q, s = fp8_weight
    if (q.dtype != ops.FP8_DTYPE or tuple(q.shape) != tuple(weight.shape) or s.dtype != torch.float32
            or tuple(s.shape) != (weight.shape[0], weight.shape[2]) or q.device != weight.device):
        raise ValueError(f"fp8_weight must be (float8_e4m3fn {tuple(weight.shape)}, fp32 "
                         f"{(weight.shape[0], weight.shape[2])}) on {weight.device}")
    return q, s


def silu_jagged_fp8(
    seq_offsets: torch.Tensor,
    Jagged: torch.Tensor,
    max_seq_len: int,
    K: int,
    Silu_Jagged: torch.Tensor,
    Silu_Jagged_fp8: torch.Tensor,
    Silu_Jagged_Scale: torch.Tensor,
    kernel: KernelType = KernelType.HIP,
) -> torch.Tensor:
    """kernels/moe_fp8.py:31-74: ``silu(Jagged)`` quantised per row; returns the fp8 tensor.  Like
    the reference's PyTorch path, the three buffer arguments are not written."""
    require_hip_kernel(kernel, "silu_jagged_fp8")
    q, _ = ops.quant_rows_fp8(Jagged, apply_silu=True)
    return q


def bmm_weight_rowwise_quant_fp8(weight: torch.Tensor, kernel: KernelType = KernelType.HIP) -> torch.Tensor:
    """kernels/moe_fp8.py:77-95: weight [E, D_in, D_out], one scale per (expert, output column)
    from the amax over D_in; returns the fp8 weight in the same [E, D_in, D_out] layout."""
    require_hip_kernel(kernel, "bmm_weight_rowwise_quant_fp8")
    q, _ = ops.quant_rows_fp8(weight.permute(0, 2, 1), out_like_input=True)
    return q.permute(0, 2, 1)


def silu_jagged_bmm_fp8(
    seq_offsets: torch.Tensor,
    max_seq_len: int,
    jagged: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor,
    kernel: KernelType = KernelType.HIP,
    *,
    fp8_weight: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
) -> torch.Tensor:
    """kernels/moe_fp8.py:98-124 with weight [E, D_out, D_in] (kernels/pytorch/moe_fp8.py:46-75):
    ``silu(jagged)`` row-quantised, weight row-quantised, fp8 GEMM + bias.  ``fp8_weight``: the
    pair ``quantize_expert_weights(weight.permute(0, 2, 1))`` when the caller keeps it."""
    require_hip_kernel(kernel, "silu_jagged_bmm_fp8")
    ops._forward_only("silu_jagged_bmm_fp8", jagged, weight, bias)
    qa, sa = ops.quant_rows_fp8(jagged, apply_silu=True)
    qw, sw = _weight_pair(weight.permute(0, 2, 1), fp8_weight)          # rows of [E, D_out, D_in]
    return ops.grouped_gemm(seq_offsets, qa, qw, total_rows=jagged.shape[0], bias=bias,
                            scales_pow2=ops.scales_are_pow2(sa, sw), a_scale=sa, b_scale=sw, epilogue=EPI_NONE)


def silu_jagged_bmm_combine_fp8(
    max_seq_len: int,
    offsets: torch.Tensor,
    jagged: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    index: torch.Tensor,
    reverse_index: torch.Tensor,
    gating_scores: Optional[torch.Tensor] = None,
    gates_index: Optional[torch.Tensor] = None,
    activation_checkpointing: bool = False,
    has_silu: bool = True,
    kernel: KernelType = KernelType.HIP,
    *,
    fp8_weight: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
) -> torch.Tensor:
    """kernels/moe_fp8.py:127-182: (SiLU +) row-quant of the hidden, weight row-quant, fp8 grouped
    GEMM + bias, weighted merge.  weight is [E, D_in, D_out]; it is quantised on every call unless
    ``fp8_weight = quantize_expert_weights(weight)`` is handed in."""
    require_hip_kernel(kernel, "silu_jagged_bmm_combine_fp8")
    L, K = reverse_index.shape
    assert index.shape[0] == L * K == jagged.shape[0]
    qw, sw = _weight_pair(weight, fp8_weight)
    if _ag.needs_grad(jagged, weight, bias, gating_scores):   # forward in e4m3, backward in bf16
        return _ag.SiluJaggedBmmCombine.apply(offsets, jagged, weight, bias, index, reverse_index, gating_scores,
                                              gates_index, has_silu, (qw, sw), activation_checkpointing)
    qa, sa = ops.quant_rows_fp8(jagged, apply_silu=has_silu)
    bmm_out = ops.grouped_gemm(offsets, qa, qw, total_rows=jagged.shape[0], bias=bias,
                               scales_pow2=ops.scales_are_pow2(sa, sw), a_scale=sa, b_scale=sw, epilogue=EPI_NONE)
    return ops.combine(bmm_out, reverse_index, gating_scores, gates_index)


def index_select_jagged_bmm(
    max_seq_len: int,
    offsets: torch.Tensor,
    index: torch.Tensor,
    jagged: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    kernel: KernelType = KernelType.HIP,
    fp8: bool = False,
    *,
    fp8_weight: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
) -> torch.Tensor:
    """kernels/moe_fp8.py:185-248.  fp8=True: tokens quantised per row BEFORE the gather, weight
    per output row, fp8 MFMA GEMM, ``acc / (s_a x s_w)`` cast to bf16, plus bias
    (kernels/pytorch/moe_fp8.py:98-139); the weight is quantised on every call, as there, unless
    ``fp8_weight = quantize_expert_weights(weight)`` is handed in.  fp8=False: the bf16 operator."""
    require_hip_kernel(kernel, "index_select_jagged_bmm")
    assert index.ndim == 2 and index.shape[0] == jagged.shape[0]
    if not fp8:
        if _ag.needs_grad(jagged, weight, bias):
            return _ag.IndexSelectJaggedBmm.apply(offsets, index, jagged, weight, bias, None, None)
        return ops.grouped_gemm(offsets, jagged, weight, total_rows=index.numel(), row_index=index,
                                index_div=index.shape[-1], bias=bias, epilogue=EPI_NONE)
    assert jagged.dtype == weight.dtype and (bias is None or jagged.dtype == bias.dtype)
    qw, sw = _weight_pair(weight, fp8_weight)
    if _ag.needs_grad(jagged, weight, bias):
        return _ag.IndexSelectJaggedBmmFp8.apply(offsets, index, jagged, weight, bias, (qw, sw))
    qa, sa = ops.quant_rows_fp8(jagged)
    return ops.grouped_gemm(offsets, qa, qw, total_rows=index.numel(), row_index=index,
                            index_div=index.shape[-1], bias=bias, scales_pow2=ops.scales_are_pow2(sa, sw), a_scale=sa,
                            b_scale=sw, epilogue=EPI_NONE)
