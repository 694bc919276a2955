"""``SGMoE``: the sparsely gated MoE layer with the MRN router front-end, on the HIP operators.

Follows the layer of /root/reference/kernels/tests/mrn_test.py:48-368 (the fast counterpart of
``OrigSGMoEImpl``, kernels/pytorch/mrn.py:93-333): input norm, (noisy) L2-normalised-logit
router with softmax gates, dispatch, the two expert GEMMs with the weighted merge, the
load-balance loss, and the shared-expert ``addmm``.  Parameter names and shapes are the
reference's, so state_dicts interchange.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import NamedTuple, Optional, Tuple

import torch
import torch.nn.functional as F

from ..kernels import moe
from ..kernels.hip import ops
from ..kernels.hip._lib import EPI_SILU
from ..kernels.utils import KernelType
from ..utils.utils import (_compute_top_logits, _create_fused_mlp_weights, _dispatch, _noisy_logits,
                           _prob_in_top_k, _train_loss, fx_torch_zeros)


class MRNOutput(NamedTuple):
    """kernels/pytorch/mrn.py:22-25."""
    x: torch.Tensor
    loss: Optional[torch.Tensor]
    load: Optional[torch.Tensor]


@dataclass
class SGConfig:
    """kernels/pytorch/mrn.py:28-42."""
    model_d: int
    num_experts: int
    num_activated_experts: int
    loss_coef: float = 1e-2
    use_input_dtype: bool = True
    activation_checkpointing: bool = False
    enable_noisy_gating: bool = False


class SGMoE(torch.nn.Module):
    def __init__(self, input_size: int, output_size: int, group_norm: bool, num_groups: int, config: SGConfig,
                 custom_kernel: bool = True, is_train: bool = True, test_mode: bool = False) -> None:
        super().__init__()
        self.num_experts = config.num_experts
        self.k = config.num_activated_experts
        self.loss_coef = 1e-2                      # mrn_test.py:77 (the test layer fixes it)
        self.model_d = config.model_d
        self.output_size = output_size
        self.input_size = input_size
        self.is_train = is_train
        self.use_input_dtype = config.use_input_dtype
        self.enable_noisy_gating = config.enable_noisy_gating
        self.group_norm = group_norm
        self.num_groups = num_groups
        self.norm_eps = 1e-6
        assert 0 < self.k <= self.num_experts
        E, D, H, O = self.num_experts, input_size, self.model_d, output_size
        norm_dim = num_groups if group_norm else D
        self._norm_w = torch.nn.Parameter(torch.ones((norm_dim,)))
        self._norm_bias = torch.nn.Parameter(torch.zeros((norm_dim,)))
        self._experts_hidden_w = torch.nn.Parameter(_create_fused_mlp_weights(E, H, D))
        self._experts_hidden_bias = torch.nn.Parameter(torch.zeros([E, H]))
        self._experts_w = torch.nn.Parameter(_create_fused_mlp_weights(E, O, H))
        self._experts_bias = torch.nn.Parameter(torch.zeros([E, O]))
        self._w_gate = torch.nn.Parameter(torch.zeros(D, E) if self.enable_noisy_gating else torch.empty(D, E))
        if self.enable_noisy_gating:
            self._w_noise = torch.nn.Parameter(torch.zeros(D, E))
        else:
            torch.nn.init.xavier_uniform_(self._w_gate)
        self.register_buffer("mean", torch.tensor([0.0]))
        self.register_buffer("std", torch.tensor([1.0]))
        self._output_weight = torch.nn.Parameter(torch.empty((D, O)))
        torch.nn.init.xavier_uniform_(self._output_weight)
        self._k_plus = min(self.k + 1, self.num_experts)

    def _noisy_gating(self, x: torch.Tensor, train: bool, noise: Optional[torch.Tensor] = None):
        """mrn_test.py:224-283: (load, top-k gates, top-k ids, loss)."""
        clean_logits = x @ self._w_gate
        noisy = train and self.enable_noisy_gating
        if noisy:
            if noise is None:
                noise = torch.randn_like(clean_logits)
            noisy_logits, noise_stddev, _ = _noisy_logits(x, clean_logits, self._w_noise, noise)
            logits = noisy_logits
        else:
            logits = clean_logits
        k_plus = self._k_plus if (noisy and self.k < self.num_experts) else self.k
        top_logits, top_k_gates, top_k_indices = _compute_top_logits(
            logits, self.k, k_plus, x.dtype if self.use_input_dtype else logits.dtype, False, True)
        gates = torch.zeros_like(logits, dtype=top_k_gates.dtype).scatter(1, top_k_indices, top_k_gates)
        if self.k < self.num_experts and noisy:
            load = _prob_in_top_k(clean_logits, noisy_logits, noise_stddev, top_logits, self.mean, self.std, self.k)
        else:
            load = gates > 0
        if not train:
            return load, top_k_gates, top_k_indices, fx_torch_zeros([], device=top_k_gates.device, requires_grad=False)
        return load, top_k_gates, top_k_indices, _train_loss(gates, load, self.loss_coef)

    def _expert_forward(self, x, token_index, offsets, reverse_index, gate_index, gating_scores):
        """mrn_test.py:292-327 without the host-side max_seq_len."""
        if not torch.is_grad_enabled():
            # inference: SiLU in the epilogue of the first GEMM (rounded to bf16 before and after the
            # activation, as the two-operator form rounds it), no pass of its own
            hidden = ops.grouped_gemm(offsets, x, self._experts_hidden_w.permute(0, 2, 1).to(x.dtype),
                                      total_rows=gate_index.numel(), row_index=gate_index, index_div=self.k,
                                      bias=self._experts_hidden_bias.to(x.dtype), epilogue=EPI_SILU)
            return moe.silu_jagged_bmm_combine(
                0, offsets, hidden, self._experts_w.permute(0, 2, 1).to(x.dtype), self._experts_bias.to(x.dtype),
                token_index, reverse_index, gating_scores, gate_index, has_silu=False, kernel=KernelType.HIP)
        hidden = moe.index_select_jagged_bmm(
            0, offsets, gate_index.view(-1, self.k), x, self._experts_hidden_w.permute(0, 2, 1).to(x.dtype),
            self._experts_hidden_bias.to(x.dtype), kernel=KernelType.HIP)
        return moe.silu_jagged_bmm_combine(
            0, offsets, hidden, self._experts_w.permute(0, 2, 1).to(x.dtype), self._experts_bias.to(x.dtype),
            token_index, reverse_index, gating_scores, gate_index, kernel=KernelType.HIP)

    def router_forward(self, x: torch.Tensor, train: bool, noise: Optional[torch.Tensor] = None) -> MRNOutput:
        load, top_k_gates, top_k_indices, loss = self._noisy_gating(x, train, noise)
        r = ops.route_from_topk(top_k_indices, self.num_experts)
        y = self._expert_forward(x, r["token_index"], r["offsets"], r["reverse_index"], r["gate_index"],
                                 top_k_gates)
        hit = load > 0 if load.dtype != torch.bool else load
        return MRNOutput(y, loss, hit.sum(0) / hit.sum())

    def forward(self, x: torch.Tensor, noise: Optional[torch.Tensor] = None) -> MRNOutput:
        """kernels/pytorch/mrn.py:298-333: norm -> router + experts -> shared-expert addmm."""
        if self.group_norm:       # as the reference calls it: one affine pair per group
            x_norm = F.group_norm(x.view(-1, self.num_groups, self.input_size // self.num_groups),
                                  num_groups=self.num_groups, weight=self._norm_w, bias=self._norm_bias,
                                  eps=self.norm_eps).view(-1, self.input_size)
        else:
            x_norm = F.layer_norm(x, (x.shape[-1],), self._norm_w, self._norm_bias, self.norm_eps)
        x_norm = x_norm.to(x.dtype) if self.use_input_dtype else x_norm
        out = self.router_forward(x_norm, self.training, noise)
        y = torch.addmm(out.x.to(x.dtype), x, self._output_weight.to(x.dtype))
        return MRNOutput(y, out.loss, out.load)
