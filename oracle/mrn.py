"""SGMoE / MRN layer oracle: the original dense-dispatch formulation.

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

Restates /root/reference/kernels/pytorch/mrn.py:52-333 (``OrigDispatcherImpl``,
``OrigSGMoEImpl``) as functions of a parameter dict: L2-normalised-logit router with stable
descending sort and softmax gates (:218-274), dispatch by non-zero gates (:52-67), per-expert
``F.linear`` + SiLU + ``F.linear`` (:280-295), fp32 ``index_add`` combine (:69-90), CV^2
load-balance loss (:182-185, :270-273) and the shared-expert ``addmm`` (:331).

Pinned by tests/test_oracle_mrn.py: gate rows against a direct softmax, the dispatcher's
per-expert row sets against the permutation of oracle.routing, and the whole router
against the operator-level oracle (oracle.moe) driven by the same routing -- an independent
formulation of the same layer (the comparison the reference's own mrn_test.py makes).
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch
import torch.nn.functional as F
from torch.distributions import Normal


def cv_squared(x: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """mrn.py:182-185."""
    if x.shape[0] == 1:
        return torch.tensor([0]).to(x.dtype)
    return x.float().var() / (x.float().mean() ** 2 + eps)


def prob_in_top_k(clean, noisy, noise_stddev, noisy_top_values, k: int) -> torch.Tensor:
    """mrn.py:187-216 with mean 0, std 1."""
    batch, m = clean.size(0), noisy_top_values.size(1)
    flat = noisy_top_values.flatten()
    pos_in = torch.arange(batch) * m + k
    thr_in = flat.gather(0, pos_in).unsqueeze(1)
    is_in = noisy > thr_in
    thr_out = flat.gather(0, pos_in - 1).unsqueeze(1)
    normal = Normal(torch.tensor([0.0]), torch.tensor([1.0]), validate_args=False)
    return torch.where(is_in, normal.cdf((clean - thr_in) / noise_stddev), normal.cdf((clean - thr_out) / noise_stddev))


def noisy_gating(p: Dict[str, torch.Tensor], x: torch.Tensor, k: int, train: bool, noisy: bool,
                 noise: Optional[torch.Tensor] = None, noise_eps: float = 1e-2,
                 post_softmax: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """mrn.py:218-274 -> (gates [T, E], loss before loss_coef)."""
    E = p["_w_gate"].shape[1]
    k_plus = min(k + 1, E)
    clean = x @ p["_w_gate"]
    if train and noisy:
        stddev = F.softplus(x @ p["_w_noise"]) + noise_eps
        noisy_logits = clean + noise * stddev
        logits = noisy_logits
    else:
        logits = clean
    logits = F.normalize(logits, dim=1)
    sorted_logits, sorted_idx = logits.sort(descending=True, dim=1, stable=True)
    top_logits = sorted_logits[:, :k_plus]
    top_idx = sorted_idx[:, :k]
    if post_softmax and k > 1:
        top_gates = F.softmax(sorted_logits[:, :k], dim=1)
    else:
        top_gates = F.softmax(sorted_logits, dim=1)[:, :k]
    top_gates = top_gates.to(x.dtype)
    gates = torch.zeros_like(logits).to(top_gates.dtype).scatter(1, top_idx, top_gates)
    if k < E and train and noisy:
        load = prob_in_top_k(clean, noisy_logits, stddev, top_logits, k).sum(0)
    else:
        load = (gates > 0).sum(0)
    if not train:
        return gates, torch.zeros([])
    return gates, cv_squared(gates.sum(0)) + cv_squared(load)


def dispatch_order(gates: torch.Tensor):
    """mrn.py:53-62: (batch_index [R], expert-sorted non-zero gates [R, 1], rows per expert)."""
    nz = torch.nonzero(gates)
    sorted_experts, order = nz.sort(0)
    expert_index = sorted_experts[:, 1:2]
    batch_index = nz[order[:, 1], 0]
    sizes = (gates > 0).sum(0).tolist()
    nonzero_gates = gates[batch_index].gather(1, expert_index)
    return batch_index, nonzero_gates, sizes


def router_forward(p: Dict[str, torch.Tensor], x: torch.Tensor, k: int, train: bool, noisy: bool = False,
                   noise: Optional[torch.Tensor] = None, loss_coef: float = 1e-2):
    """mrn.py:276-296 -> (y [T, O], loss, load fractions [E])."""
    gates, loss = noisy_gating(p, x, k, train, noisy, noise)
    loss = loss * loss_coef
    batch_index, nonzero_gates, sizes = dispatch_order(gates)
    inputs = x[batch_index].split(sizes, dim=0)
    E = gates.shape[1]
    hidden = [F.silu(F.linear(inputs[e], p["_experts_hidden_w"][e], p["_experts_hidden_bias"][e])) for e in range(E)]
    outs = [F.linear(hidden[e], p["_experts_w"][e], p["_experts_bias"][e]) for e in range(E)]
    stitched = torch.cat(outs, 0).mul(nonzero_gates)
    y = torch.zeros(x.shape[0], stitched.shape[1], dtype=torch.float32).index_add(
        0, batch_index, stitched.float()).to(stitched.dtype)
    return y, loss, (gates > 0).sum(0) / (gates > 0).sum()


def sgmoe_forward(p: Dict[str, torch.Tensor], x: torch.Tensor, k: int, train: bool, noisy: bool = False,
                  noise: Optional[torch.Tensor] = None, norm_eps: float = 1e-6, loss_coef: float = 1e-2):
    """mrn.py:298-333 with layer norm."""
    x_norm = F.layer_norm(x, (x.shape[-1],), p["_norm_w"], p["_norm_bias"], norm_eps).to(x.dtype)
    y, loss, load = router_forward(p, x_norm, k, train, noisy, noise, loss_coef)
    return torch.addmm(y, x, p["_output_weight"]), loss, load
