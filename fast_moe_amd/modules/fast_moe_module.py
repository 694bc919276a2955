"""``FastMoELayer``: the MoE layer of /root/reference/modules/fast_moe_module.py:45-225
on the MI355X HIP back-end.

Constructor arguments, parameter names / shapes / dtypes (so state_dicts
interchange) and ``forward(x, num_experts_per_tok)`` are the reference's.  The
gate (Linear + softmax) stays a torch call; everything after it -- top-k, gate
renormalisation, routing tensors, both expert GEMMs, SiLU and the weighted
merge -- runs in libfastmoe_hip.so with no host synchronisation (the reference
syncs once for ``max_seq_len``, fast_moe_module.py:135).
"""
from __future__ import annotations

from typing import Dict

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.autograd.profiler import record_function

from ..kernels.hip import ops
from ..kernels.hip._lib import EPI_NONE, EPI_SILU
from ..kernels.utils import KernelType, require_hip_kernel
from ..utils.utils import _create_fused_mlp_weights


class GatingNetwork(nn.Module):
    """fast_moe_module.py:21-27."""

    def __init__(self, input_dim: int, num_experts: int) -> None:
        super().__init__()
        self.gate = nn.Linear(input_dim, num_experts)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return F.softmax(self.gate(x), dim=2)


class FastMoELayer(nn.Module):
    def __init__(
        self,
        input_dim: int,
        hidden_dim: int,
        output_dim: int,
        num_experts: int,
        kernel: KernelType = KernelType.HIP,
        dtype: torch.dtype = torch.bfloat16,
    ) -> None:
        super().__init__()
        self.input_dim: int = input_dim
        self.hidden_dim: int = hidden_dim
        self.output_dim: int = output_dim
        self.num_experts: int = num_experts
        self.kernel: KernelType = kernel
        self.dtype: torch.dtype = dtype

        self.gate = GatingNetwork(input_dim, num_experts)
        self._experts_hidden_w = nn.Parameter(
            _create_fused_mlp_weights(num_experts, hidden_dim, input_dim).to(dtype=dtype))
        self._experts_hidden_bias = nn.Parameter(torch.zeros([num_experts, hidden_dim], dtype=dtype))
        self._experts_w = nn.Parameter(
            _create_fused_mlp_weights(num_experts, output_dim, hidden_dim).to(dtype=dtype))
        self._experts_bias = nn.Parameter(torch.zeros([num_experts, output_dim], dtype=dtype))

    def route(self, x: torch.Tensor, num_experts_per_tok: int) -> Dict[str, torch.Tensor]:
        """fast_moe_module.py:93-144 in one library call on the gate probabilities."""
        scores = self.gate(x).reshape(-1, self.num_experts)
        return ops.route_topk(scores, num_experts_per_tok, renorm=True)

    def quantized_expert_weights(self, refresh: bool = False) -> Dict[str, torch.Tensor]:
        """Row-quantised e4m3 copies of both expert weight tensors in the layout the fp8 operators
        take as ``fp8_weight`` ([E, D_in, D_out] views of K-contiguous bytes) with their [E, D_out]
        multiplier scales.  Kept beside the parameters (not in the state_dict) until a parameter
        is updated in place or replaced; the reference re-quantises on every call
        (kernels/pytorch/moe_fp8.py:111).  Writes through ``param.data`` do not move the version
        counter the cache watches: pass ``refresh=True`` after such an update."""
        from ..kernels.moe_fp8 import cached_quantize_expert_weights, weight_quant_cache
        if refresh:
            weight_quant_cache.invalidate(self._experts_hidden_w)
            weight_quant_cache.invalidate(self._experts_w)
        qh, sh = cached_quantize_expert_weights(self._experts_hidden_w.permute(0, 2, 1))
        qo, so = cached_quantize_expert_weights(self._experts_w.permute(0, 2, 1))
        return {"hidden_w": qh, "hidden_scale": sh, "out_w": qo, "out_scale": so}

    def _forward_with_grad(self, x: torch.Tensor, k: int) -> torch.Tensor:
        """The two-operator form of fast_moe_module.py:146-186 on the differentiable HIP operators
        (same values as ``forward``: the fused SiLU epilogue rounds where this form rounds).  The
        routing integers come from the library; the K gate values are re-derived from the gate
        probabilities with torch ops so that the gate network receives its gradient
        (fast_moe_module.py:93-105: mask, then L1 normalisation)."""
        from ..kernels import moe
        if x.dtype not in (torch.bfloat16, torch.float32):
            raise NotImplementedError(f"FastMoELayer: the HIP kernels take bf16 or fp32 activations, got {x.dtype}")
        original_shape = x.shape
        scores = self.gate(x).reshape(-1, self.num_experts)
        r = ops.route_topk(scores.detach(), k, renorm=True)
        picked = scores.gather(1, r["topk_idx"])
        gates = picked / picked.sum(dim=1, keepdim=True).clamp_min(1e-12)
        x_flat = x.reshape(-1, self.input_dim)
        T = x_flat.shape[0]
        hidden = moe.index_select_jagged_bmm(
            0, r["offsets"], r["gate_index"].view(T, k), x_flat,
            self._experts_hidden_w.permute(0, 2, 1).to(x.dtype), self._experts_hidden_bias.to(x.dtype))
        y = moe.silu_jagged_bmm_combine(
            0, r["offsets"], hidden, self._experts_w.permute(0, 2, 1).to(x.dtype),
            self._experts_bias.to(x.dtype), r["token_index"], r["reverse_index"], gates, r["gate_index"],
            has_silu=True)
        return y.view(original_shape[0], original_shape[1], self.output_dim)

    def forward(self, x: torch.Tensor, num_experts_per_tok: int) -> torch.Tensor:
        require_hip_kernel(self.kernel, "FastMoELayer.forward")
        if torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in self.parameters())):
            return self._forward_with_grad(x, num_experts_per_tok)
        if x.dtype not in (torch.bfloat16, torch.float32):
            raise NotImplementedError(f"FastMoELayer: the HIP kernels take bf16 or fp32 activations, got {x.dtype}")
        original_shape = x.shape
        k = num_experts_per_tok
        r = self.route(x, k)
        with record_function("## expert_forward##"):
            x_flat = x.reshape(-1, self.input_dim)
            # GEMM1 with SiLU in the epilogue: the hidden is rounded to bf16 before and after the
            # activation, exactly as the two-operator form of fast_moe_module.py:162-184 rounds it
            hidden = ops.grouped_gemm(
                r["offsets"], x_flat, self._experts_hidden_w.permute(0, 2, 1).to(x.dtype),
                total_rows=x_flat.shape[0] * k, row_index=r["gate_index"], index_div=k,
                bias=self._experts_hidden_bias.to(x.dtype), epilogue=EPI_SILU)
            out_rows = ops.grouped_gemm(
                r["offsets"], hidden, self._experts_w.permute(0, 2, 1).to(x.dtype),
                total_rows=hidden.shape[0], bias=self._experts_bias.to(x.dtype), epilogue=EPI_NONE)
            y = ops.combine(out_rows, r["reverse_index"], r["gates"], r["gate_index"])
        return y.view(original_shape[0], original_shape[1], self.output_dim)
